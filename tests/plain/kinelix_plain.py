"""Plain Kinelix decoder: whole sequences, no cache, one function per mechanism.

Pre-norm layers with layer norms (a weight, no bias) and a learned scale per channel on every sublayer's
output.  Mixers: the Mamba-2 recurrence (a scalar decay per head, inputs behind one short convolution, a gated
norm in groups), the gated delta rule with a decay per head, and latent attention without positions whose
softmax has a sink per head; a latent attention layer may read the latent rows of an earlier layer.
Feed-forwards: a gated dense layer, or experts behind a sigmoid router with a correction that enters the
choice only and a choice limited to the best groups of experts.  The logits pass a soft cap.

Everything runs on the CPU in float64 from a configuration (the dict of config.json) and a dict of tensors
by checkpoint name.  Nothing of the product package is imported.

`rnd`: where given, applied to the activations that an engine with bfloat16 activations keeps in bfloat16
between two operations; norms, scores, routers, recurrences and the residual stream stay exact.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def _same(t):
    return t


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).to(torch.bfloat16).to(t.dtype)


# ------------------------------------------------------------------------ small functions
def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w over the last axis, var the mean of the squared deviations."""
    mu = x.mean(-1, keepdim=True)
    dev = x - mu
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * w


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(x, taps, bias=None):
    """y[t, c] = sum_j taps[c, j] x[t - (K - 1) + j, c] (+ bias[c]); zeros stand before the first token.
    x [T, C], taps [C, K]: the last column meets the token itself."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x])
    y = torch.zeros(T, C, dtype=x.dtype)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y if bias is None else y + bias


# ------------------------------------------------------------------------------ mixers
def mamba2(n, W, m, eps, rnd=_same):
    """n [T, d] -> [T, d].  W: the mixer's tensors by their short names."""
    T = n.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = n @ W["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = rnd(silu(causal_conv(rnd(xbc), W["conv"], W["conv.b"])))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W["dt_bias"])                                  # [T, H]
    decay = torch.exp(-torch.exp(W["A_log"]) * dt)                    # [T, H]
    y = torch.zeros(T, H, P, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = decay[t, h] * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + W["D"][h] * x[t, h]
    y = y.reshape(T, inner) * silu(rnd(z))
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W["norm"]
    return rnd(y) @ W["o"].T


def gated_delta(n, W, m, eps, rnd=_same):
    """n [T, d] -> [T, d]: the gated delta rule with one decay per head."""
    T = n.shape[0]
    H, Hk, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(silu(causal_conv(rnd(n @ W["q"].T), W["q.conv"]))).view(T, Hk, D)
    k = rnd(silu(causal_conv(rnd(n @ W["k"].T), W["k.conv"]))).view(T, Hk, D)
    v = rnd(silu(causal_conv(rnd(n @ W["v"].T), W["v.conv"]))).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(n @ W["b"].T)                                 # [T, H]
    g = torch.exp(-torch.exp(W["A_log"]) * softplus(n @ W["a"].T + W["dt_bias"]))        # [T, H]
    o = torch.zeros(T, H, Dv, dtype=F64)
    for h in range(H):
        a = h // (H // Hk)
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = g[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, a])
            S = S + torch.outer(k[t, a], u)
            o[t, h] = S.T @ q[t, a]
    o = unit_rms(o, eps) * W["norm"]
    o = o.reshape(T, H * Dv) * silu(rnd(n @ W["g"].T))
    return rnd(o) @ W["o"].T


def latent_rows(n, W, eps, rnd=_same):
    """The latent row of every token: the normed narrow projection, c [T, rank]."""
    return rnd(unit_rms(n @ W["dkv"].T, eps) * W["dkv.norm"])


def latent_attention(n, c, W, m, rnd=_same):
    """n [T, d], c [T, rank] (this layer's latent rows or an earlier layer's) -> [T, d].  Keys and values are
    expanded from c by this layer's own matrices; the softmax's denominator also holds exp(sink_h)."""
    T = n.shape[0]
    H, dk, dv, scale = m["heads"], m["dim"], m["vdim"], m["scale"]
    q = rnd(n @ W["q"].T).view(T, H, dk)
    k = rnd(c @ W["uk"].T).view(T, H, dk)
    v = rnd(c @ W["uv"].T).view(T, H, dv)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    mask = torch.arange(T)[None, :] > torch.arange(T)[:, None]
    s = s.masked_fill(mask[None], -math.inf)
    top = torch.maximum(s.max(-1).values, W["sink"][:, None])                  # [H, T]
    e = torch.exp(s - top[..., None])
    p = e / (e.sum(-1) + torch.exp(W["sink"][:, None] - top))[..., None]
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(T, H * dv)
    return rnd(o) @ W["o"].T


# ------------------------------------------------------------------------ feed-forwards
def dense_ff(n, W, rnd=_same):
    return rnd(silu(n @ W["gate"].T) * (n @ W["up"].T)) @ W["down"].T


def route(n, W, spec, margins_out=None):
    """ids [T, top] and weights [T, top].  Scores are sigmoid(W_router n); the choice runs on score + correction,
    only inside the groups.keep groups whose two largest choice scores have the largest sum; the weights are the
    chosen experts' plain scores times router.scale, not renormalised.  Ties go to the lower index.
    margins_out: a list that receives, per token, the smaller of two gaps, each as a share of the root mean square of
    all the sequence's choice scores about their mean: between the last kept group's score and the first dropped one's,
    and between the last chosen expert's choice score and the first one left out inside the kept groups (infinite
    where nothing is left out)."""
    r = spec["router"]
    E, top = r["experts"], r["top"]
    count, keep = r["groups"]["count"], r["groups"]["keep"]
    s = torch.sigmoid(n @ W["router"].T)                                 # [T, E]
    choice = s + W["correction"]
    T = n.shape[0]
    per = E // count
    ids = torch.zeros(T, top, dtype=torch.long)
    margins = torch.full((T,), math.inf, dtype=F64)
    spread = (choice - choice.mean()).pow(2).mean().sqrt().clamp_min(1e-30)
    for t in range(T):
        grp = []
        for g in range(count):
            vals = sorted(choice[t, g * per:(g + 1) * per].tolist(), reverse=True)
            grp.append(sum(vals[:2]))
        kept = sorted(range(count), key=lambda g: (-grp[g], g))[:keep]
        allowed = [e for e in range(E) if e // per in kept]
        order = sorted(allowed, key=lambda e: (-choice[t, e].item(), e))
        ids[t] = torch.tensor(order[:top])
        by_score = sorted(grp, reverse=True)
        if keep < count:
            margins[t] = min(margins[t], (by_score[keep - 1] - by_score[keep]) / spread)
        if top < len(order):
            margins[t] = min(margins[t], (choice[t, order[top - 1]] - choice[t, order[top]]) / spread)
    if margins_out is not None:
        margins_out.append(margins)
    wts = torch.gather(s, 1, ids) * r["scale"]
    return ids, wts


def moe_ff(n, W, spec, rnd=_same, margins_out=None):
    T, d = n.shape
    ids, wts = route(n, W, spec, margins_out)
    out = torch.zeros(T, d, dtype=F64)
    for t in range(T):
        for e, w in zip(ids[t].tolist(), wts[t]):
            a = rnd(silu(n[t] @ W[f"e{e}.gate"].T) * (n[t] @ W[f"e{e}.up"].T))
            out[t] = out[t] + w * (a @ W[f"e{e}.down"].T)
    return out


# ------------------------------------------------------------------------------- model
def _sub(weights, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: dict, tokens, rnd=_same, on_layer=None, margins_out=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  on_layer(i, x): called with the residual stream after every layer.
    margins_out: see route()."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = weights["embed"].to(F64)[tokens] * cfg["embedding"]["scale"]
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        W = _sub(weights, f"l{i}.mix.")
        n = rnd(layer_norm(x, weights[f"l{i}.norm1"].to(F64), eps))
        if layer["type"] == "mamba2":
            y = mamba2(n, W, m, eps, rnd)
        elif layer["type"] == "delta":
            y = gated_delta(n, W, m, eps, rnd)
        else:
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_rows(n, W, eps, rnd)
                src = i
            y = latent_attention(n, latents[src], W, m, rnd)
        x = x + y * weights[f"l{i}.ls1"].to(F64)
        spec = layer.get("mlp")
        if spec is not None:
            n = rnd(layer_norm(x, weights[f"l{i}.norm2"].to(F64), eps))
            Wf = _sub(weights, f"l{i}.mlp.")
            y = dense_ff(n, Wf, rnd) if spec["kind"] == "dense" else moe_ff(n, Wf, spec, rnd, margins_out)
            x = x + y * weights[f"l{i}.ls2"].to(F64)
        if on_layer is not None:
            on_layer(i, x)
    h = rnd(layer_norm(x, weights["final.norm"].to(F64), eps))
    logits = h @ weights["head"].to(F64).T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
