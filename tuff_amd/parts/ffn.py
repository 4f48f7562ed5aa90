"""Feed-forwards.

GatedMLP: W_down (act(W_gate h + b_g) * (W_up h + b_u)) + b_d with act silu or the tanh form of gelu, biases optional.
DenseMLP: W_down act(W_up h + b_u) + b_d without a gate, act the square of relu or any other of the row activations.
MoE: routed experts W_down act(W_up x) chosen per token by a router, and an optional shared expert.

SwiGLU feed-forward: W_down (silu(W_gate h) * (W_up h)), silu(g) = g / (1 + exp(-g)).
Reference: src/lfm25_gpu.cu:583-618 (gate and up in one pass with the activation fused),
src/lfm25_engine.c:412-419.  Gate and up are one product; with bfloat16 weights their rows are
interleaved and the activation is the product's epilogue.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import FEED_FORWARDS, FeedForward, Runtime, WeightDecl
from .linear import Linear


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    records_portions = True
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, ffn_dim: int, *, names: dict[str, str],
                 aliases: dict[str, tuple] | None = None):
        """names: checkpoint names of 'gate' [F, d], 'up' [F, d], 'down' [d, F]."""
        self.d, self.F = int(hidden_size), int(ffn_dim)
        self._names, self._al = dict(names), aliases or {}
        self._make(self.F)
        self._decls = self.gate_up.weight_decls() + self.down.weight_decls()

    def _make(self, width: int) -> None:
        names, al = self._names, self._al
        self.gate_up = Linear([names["gate"], names["up"]], self.d, [width, width],
                              aliases=[al.get("gate", ()), al.get("up", ())], swiglu_pair=True)
        self.down = Linear(names["down"], width, self.d, aliases=[al.get("down", ())])
        self.width = width

    def weight_decls(self):
        return self._decls

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        names = self._names
        g, u, dn = (weights[names[k]] for k in ("gate", "up", "down"))
        if self.F % 8 and all(t.dtype == torch.bfloat16 for t in (g, u, dn)):
            # The bfloat16 matrix kernels read 16 bytes at a time along the inner size.  A width that is
            # no multiple of 8 is filled up with zero rows of gate and up (silu(0) * 0 = 0, exactly) and
            # zero columns of down: the same function.
            pad = -self.F % 8
            weights = dict(weights)
            weights[names["gate"]] = torch.cat([g, g.new_zeros(pad, self.d)])
            weights[names["up"]] = torch.cat([u, u.new_zeros(pad, self.d)])
            weights[names["down"]] = torch.cat([dn, dn.new_zeros(self.d, pad)], dim=1).contiguous()
            self._make(self.F + pad)
        self.gate_up.bind(weights, rt)
        self.down.bind(weights, rt)

    def forward(self, h, ctx, residual, next_norm=None) -> None:
        if self.gate_up.interleaved:
            act = self.gate_up.forward(h, swiglu=True)          # silu(gate) * up in the product's epilogue
        else:
            gu = self.gate_up.forward(h)
            act = self.rt.empty(h.shape[0], self.width, dtype=gu.dtype)
            ops.swiglu(gu, act)
        self.down.forward(act, accumulate_into=residual, next_norm=next_norm)


@FEED_FORWARDS.register("gated")
class GatedMLP(FeedForward):
    """W_down (act(W_gate h + b_gate) * (W_up h + b_up)) + b_down.  activation: "silu" or "gelu_tanh"
    (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))), or "swish_clamp": with g = min(W_gate h, limit) and
    u = clamp(W_up h, -limit, limit) the product is g sigmoid(alpha g) (u + 1).  names: 'gate', 'up' [F, d],
    'down' [d, F] and, with bias=True, 'gate.b', 'up.b' [F], 'down.b' [d]."""
    graph_safe = True
    records_portions = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, ffn_dim: int, *, names: dict[str, str], activation: str = "gelu_tanh",
                 bias: bool = False, limit: float = 0.0, alpha: float = 1.0):
        if activation not in ("silu", "gelu_tanh", "swish_clamp"):
            raise ValueError(f"unknown activation '{activation}'")
        if activation == "swish_clamp" and not limit > 0:
            raise ValueError("the clamped activation needs a positive limit")
        self.d, self.F, self.activation, self.has_bias = int(hidden_size), int(ffn_dim), activation, bool(bias)
        self.limit, self.alpha = float(limit), float(alpha)
        self._names = dict(names)
        self._make(self.F)
        self._decls = self.gate_up.weight_decls() + self.down.weight_decls()
        if self.has_bias:
            self._decls += [WeightDecl(names["gate.b"], (self.F,), "normal"), WeightDecl(names["up.b"], (self.F,), "normal")]

    def _make(self, width: int) -> None:
        n = self._names
        self.gate_up = Linear([n["gate"], n["up"]], self.d, [width, width])      # (its biases go into the activation's kernel)
        self.down = Linear(n["down"], width, self.d, bias=n["down.b"] if self.has_bias else None)
        self.width = width

    def weight_decls(self):
        return self._decls

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        n = self._names
        g, u, dn = (weights[n[k]] for k in ("gate", "up", "down"))
        if self.F % 8 and all(t.dtype == torch.bfloat16 for t in (g, u, dn)):
            # zero rows of gate and up (with zero biases: act(0) * 0 = 0) and zero columns of down: the same function
            pad = -self.F % 8
            weights = dict(weights)
            weights[n["gate"]] = torch.cat([g, g.new_zeros(pad, self.d)])
            weights[n["up"]] = torch.cat([u, u.new_zeros(pad, self.d)])
            weights[n["down"]] = torch.cat([dn, dn.new_zeros(self.d, pad)], dim=1).contiguous()
            if self.has_bias:
                for k in ("gate.b", "up.b"):
                    weights[n[k]] = torch.cat([weights[n[k]], weights[n[k]].new_zeros(pad)])
            self._make(self.F + pad)
        self.gate_up.bind(weights, rt)
        self.down.bind(weights, rt)
        self.gu_bias = None
        if self.has_bias:
            self.gu_bias = torch.cat([weights[n["gate.b"]].float(), weights[n["up.b"]].float()]).contiguous()

    def forward(self, h, ctx, residual, next_norm=None) -> None:
        gu = self.gate_up.forward(h, out_dtype=torch.float32)       # the activation reads the sums as they are, plus the biases
        act = self.rt.empty(h.shape[0], self.width)
        ops.glu(gu, act, self.activation, self.gu_bias, limit=self.limit, alpha=self.alpha)
        self.down.forward(act, accumulate_into=residual, next_norm=next_norm)


@FEED_FORWARDS.register("dense")
class DenseMLP(FeedForward):
    """W_down act(W_up h + b_up) + b_down: no gate.  activation: "relu2" (the square of relu), "silu", "gelu_tanh",
    "tanh" or "sigmoid".  names: 'up' [F, d], 'down' [d, F] and, with bias=True, 'up.b' [F], 'down.b' [d]."""
    graph_safe = True
    records_portions = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, ffn_dim: int, *, names: dict[str, str], activation: str = "relu2", bias: bool = False):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation '{activation}'")
        self.d, self.F, self.activation, self.has_bias = int(hidden_size), int(ffn_dim), activation, bool(bias)
        if activation == "sigmoid" and self.F % 8:
            raise ValueError("a width that is no multiple of 8 needs an activation with act(0) = 0")
        self._names = dict(names)
        self._make(self.F)
        self._decls = self.up.weight_decls() + self.down.weight_decls()
        if self.has_bias:
            self._decls += [WeightDecl(names["up.b"], (self.F,), "normal"), WeightDecl(names["down.b"], (self.d,), "normal")]
        #: float32 [d] once bound, or None: what the feed-forward adds to every row of its output.  A block that clears the
        #: rows its sublayers add into may leave this there instead and say so (forward(bias_preloaded=True))
        self.output_bias = None

    def _make(self, width: int) -> None:
        n = self._names
        self.up = Linear(n["up"], self.d, width)                     # (its bias goes into the activation's kernel)
        self.down = Linear(n["down"], width, self.d)               # (its bias: output_bias)
        self.width = width

    def weight_decls(self):
        return self._decls

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        n = self._names
        u, dn = weights[n["up"]], weights[n["down"]]
        if self.F % 8 and u.dtype == torch.bfloat16 and dn.dtype == torch.bfloat16:
            # zero rows of up (with a zero bias: act(0) = 0) and zero columns of down: the same function
            pad = -self.F % 8
            weights = dict(weights)
            weights[n["up"]] = torch.cat([u, u.new_zeros(pad, self.d)])
            weights[n["down"]] = torch.cat([dn, dn.new_zeros(self.d, pad)], dim=1).contiguous()
            if self.has_bias:
                weights[n["up.b"]] = torch.cat([weights[n["up.b"]], weights[n["up.b"]].new_zeros(pad)])
            self._make(self.F + pad)
        self.up.bind(weights, rt)
        self.down.bind(weights, rt)
        self.up_bias = weights[n["up.b"]].float().contiguous() if self.has_bias else None
        self.output_bias = weights[n["down.b"]].float().contiguous() if self.has_bias else None

    def forward(self, h, ctx, residual, next_norm=None, bias_preloaded: bool = False) -> None:
        u = self.up.forward(h, out_dtype=torch.float32)          # the activation reads the sums as they are, plus the bias
        act = self.rt.empty(u.shape[0], self.width)
        ops.act_rows(u, act, self.activation, bias=self.up_bias)
        if self.output_bias is None or bias_preloaded:
            self.down.forward(act, accumulate_into=residual, next_norm=next_norm)
            return
        self.down.forward(act, accumulate_into=residual)          # (the sum is not final before the bias is in)
        ops.add_bias(residual, self.output_bias)


@FEED_FORWARDS.register("moe")
class MoE(FeedForward):
    """Routed experts, each W_down act(W_up x) without biases, and an optional shared expert of the same form.

    Router logits z = W_router h are float32 products.  The `top` largest are chosen per token (the lower
    index wins a tie).  router_weights "sigmoid": a choice's weight is sigmoid(z), each on its own; "softmax":
    a softmax over the chosen.  scale_input: the weight multiplies the expert's input (sum_e expert_e(w_e h));
    else its output.  The shared expert runs for every token and is multiplied by sigmoid(W_sg h), one number a
    token (names['shared.sg'], [1, d]); without that name it is added as it is.
    names: 'router' [E, d]; 'experts': a list of (up [F, d], down [d, F]) names; optional 'shared.up',
    'shared.down', 'shared.sg'; optional 'router.b' [E], a bias on the router's logits.
    gated: an expert is W_down glu(W_gate x, W_up x) and 'experts' lists (gate, up, down) names; glu(g, u) is
    act(g) u, or, activation "swish_clamp", g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit) and
    u' = clamp(u, -limit, limit).  shared: a feed-forward of any kind that runs for every token and is added (in
    place of the built-in ungated one that shared_dim asks for).
    A limited choice (router_weights "sigmoid"; switched on by route_groups, a name 'correction' or route_scale): the
    choice runs on sigmoid(z) + correction ('correction' [E], which the weights do not see) and only inside the
    route_keep groups, of route_groups equal groups of neighbouring experts, whose two largest such scores have the
    largest sum (an expert outside them cannot be chosen, whatever its score); the weights are the chosen experts'
    sigmoid(z) times route_scale, not renormalised."""
    graph_safe = True
    records_portions = True

    def __init__(self, hidden_size: int, num_experts: int, top: int, expert_dim: int, *, names: dict,
                 activation: str = "relu2", router_weights: str = "sigmoid", scale_input: bool = True,
                 shared_dim: int = 0, gated: bool = False, limit: float = 0.0, alpha: float = 1.0,
                 shared: FeedForward | None = None, route_groups: int = 0, route_keep: int = 0, route_scale: float = 1.0):
        self.d, self.E, self.top, self.F = int(hidden_size), int(num_experts), int(top), int(expert_dim)
        if not 1 <= self.top <= self.E:
            raise ValueError(f"top {self.top} of {self.E} experts")
        self.has_correction = "correction" in names
        self.route_scale = float(route_scale)
        self.route_groups, self.route_keep = int(route_groups), int(route_keep)
        if not self.route_groups and (self.has_correction or self.route_scale != 1.0):
            self.route_groups = self.route_keep = 1              # one group of all experts, kept: the choice is not limited
        if self.route_groups:
            G, keep = self.route_groups, self.route_keep
            if router_weights != "sigmoid" or "router.b" in names:
                raise ValueError("a limited choice goes with sigmoid weights and no bias on the logits")
            if not 1 <= G <= 64 or self.E % G or not 1 <= keep <= G or self.top > keep * (self.E // G):
                raise ValueError(f"top {self.top} among {keep} of {G} groups of {self.E} experts")
        if activation not in ("relu2", "silu", "gelu_tanh", "swish_clamp"):
            raise ValueError(f"unknown activation '{activation}'")
        self.gated, self.limit, self.alpha = bool(gated), float(limit), float(alpha)
        if activation == "swish_clamp" and (not self.gated or not self.limit > 0):
            raise ValueError("the clamped activation is for gated experts and needs a positive limit")
        self.activation, self.router_weights, self.scale_input = activation, router_weights, bool(scale_input)
        self.names = dict(names)
        if len(self.names["experts"]) != self.E or any(len(e) != (3 if self.gated else 2) for e in self.names["experts"]):
            raise ValueError("one (up, down) pair of names per expert ((gate, up, down) for gated experts)")
        if shared is not None and shared_dim:
            raise ValueError("either a shared feed-forward of its own or shared_dim")
        self.shared = shared
        self.has_router_bias = "router.b" in self.names
        self.Fs = int(shared_dim)
        self.shared_gate = self.Fs > 0 and "shared.sg" in self.names
        self.shared_up = self.shared_down = None
        if self.Fs:
            self._make_shared(self.Fs)

    def _make_shared(self, width: int) -> None:
        self.shared_up = Linear(self.names["shared.up"], self.d, width)
        self.shared_down = Linear(self.names["shared.down"], width, self.d)

    def weight_decls(self):
        decls = [WeightDecl(self.names["router"], (self.E, self.d), "normal", role="projection")]
        if self.shared_gate:
            decls.append(WeightDecl(self.names["shared.sg"], (1, self.d), "normal", role="projection"))
        if self.has_router_bias:
            decls.append(WeightDecl(self.names["router.b"], (self.E,), "normal"))
        if self.has_correction:
            decls.append(WeightDecl(self.names["correction"], (self.E,), "normal"))
        for e in self.names["experts"]:
            decls += [WeightDecl(n, (self.F, self.d), "normal", role="projection") for n in e[:-1]]
            decls.append(WeightDecl(e[-1], (self.d, self.F), "normal", role="projection"))
        if self.shared is not None:
            decls += self.shared.weight_decls()
        if self.Fs:
            decls += [WeightDecl(self.names["shared.up"], (self.Fs, self.d), "normal", role="projection"),
                      WeightDecl(self.names["shared.down"], (self.d, self.Fs), "normal", role="projection")]
        return decls

    def kernel_modules(self):
        return ["moe", "elementwise"] + (self.shared.kernel_modules() if self.shared is not None else [])

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        # the router's rows (and the shared expert's gate row behind them) stay float32: their products decide
        rows = [weights[self.names["router"]]] + ([weights[self.names["shared.sg"]]] if self.shared_gate else [])
        self.router_w = torch.cat([r.to(torch.float32).reshape(-1, self.d) for r in rows]).contiguous()
        self.router_b = weights[self.names["router.b"]].to(torch.float32).contiguous() if self.has_router_bias else None
        self.correction = weights[self.names["correction"]].to(torch.float32).contiguous() if self.has_correction else None
        ups = [weights[e[-2]] for e in self.names["experts"]]
        gates = [weights[e[0]] for e in self.names["experts"]] if self.gated else None
        downs = [weights[e[-1]] for e in self.names["experts"]]
        self.grouped = ops.moe_grouped_supported(ups[0].dtype, self.d, self.F, self.E) and rt.dtype == torch.bfloat16
        if self.grouped:
            # the matrix cores' order, an expert after the other; a gated expert's gate and up rows take turns
            if self.gated:
                ups = [ops.interleave_gate_up(g, u) for g, u in zip(gates, ups)]
            self.up_tiles, self.down_tiles = ops.tile_experts(ups), ops.tile_experts(downs)
        else:
            if self.gated:
                ups = [torch.cat([g, u]) for g, u in zip(gates, ups)]        # an expert's gate rows, then its up rows
            self.w_up = torch.stack(ups).contiguous()                # [E, F or 2 F, d]
            self.w_down = torch.stack(downs).contiguous()            # [E, d, F]
        if self.shared is not None:
            self.shared.bind(weights, rt)
        if self.Fs:
            up, down = weights[self.names["shared.up"]], weights[self.names["shared.down"]]
            if self.Fs % 8 and up.dtype == torch.bfloat16 and down.dtype == torch.bfloat16:
                pad = -self.Fs % 8
                weights = dict(weights)
                weights[self.names["shared.up"]] = torch.cat([up, up.new_zeros(pad, self.d)])
                weights[self.names["shared.down"]] = torch.cat([down, down.new_zeros(self.d, pad)], dim=1).contiguous()
                self._make_shared(self.Fs + pad)
            self.shared_up.bind(weights, rt)
            self.shared_down.bind(weights, rt)

    def forward(self, h, ctx, residual) -> None:
        T = h.shape[0]
        z = torch.empty(T, self.router_w.shape[0], dtype=torch.float32, device=h.device)        # [T, E (+ 1)]
        ids = torch.empty(T, self.top, dtype=torch.int32, device=h.device)
        wts = torch.empty(T, self.top, dtype=torch.float32, device=h.device)
        ops.moe_router(h, self.router_w, z, ids, wts, E=self.E, top=self.top, weights=self.router_weights, bias=self.router_b,
                       correction=self.correction, groups=self.route_groups, keep=self.route_keep, scale=self.route_scale)
        form = dict(activation=self.activation, scale_input=self.scale_input, gated=self.gated, limit=self.limit, alpha=self.alpha)
        if self.grouped:
            ops.moe_experts_grouped(h, self.up_tiles, self.down_tiles, ids, wts, residual, F=self.F, **form)
        else:
            ops.moe_experts(h, self.w_up, self.w_down, ids, wts, residual, **form)
        if self.shared is not None:
            kw = {"next_norm": None} if self.shared.adds_once_through_linear else {}
            self.shared.forward(h, ctx, residual, **kw)
        if self.Fs:
            a = self.shared_up.forward(h)
            # the gate is one number a token and the second product is linear: it goes onto the activations
            if self.shared_gate:
                ops.act_rows(a, a, self.activation, row_gate=z, gate_col=self.E, gate_activation="sigmoid")
            else:
                ops.act_rows(a, a, self.activation)
            self.shared_down.forward(a, accumulate_into=residual)
