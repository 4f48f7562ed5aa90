"""Plain Loluzen decoder: whole sequences, no cache, one function per mechanism.

Layers are "sandwiched": a sublayer's output is normed before it joins the residual stream,
x <- x + m * norm_after(sublayer(norm_before(x))).  Mixers: a pair of mixers side by side (grouped attention
with biases, a logarithmic distance penalty, softmax weights mixed between the heads and a gate per head;
beside it a gated linear recurrence whose forget gate also sets the write strength), and grouped attention
behind short causal convolutions with per-head norms, a partial rotation of neighbouring pairs with scaled
frequencies and a gate per head.  Feed-forward: W_down relu(W_up n + b)^2 + b.  A stretch of the layers may run
several times; the scaled embedding joins the stream again at the start of every later pass.

Everything runs on the CPU in float64 from a configuration (the dict of config.json) and a dict of tensors by
checkpoint name.  Nothing of the product package is imported.

`rnd`: where given, applied to the activations that an engine with bfloat16 activations keeps in bfloat16
between two operations; norms, scores, gates of the recurrence, states and the residual stream stay exact.
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
def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight lies around zero: unit_rms(x) * (1 + w)."""
    return unit_rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    """RMS norm with the weight as stored."""
    return unit_rms(x, eps) * w


def scaled_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` {factor, low, high, original}: a frequency whose
    wavelength 2 pi / f is above original / low is divided by factor, one whose wavelength is below
    original / high stays, and between the two the kept share is s = (original / wavelength - low) / (high - low):
    (1 - s) f / factor + s f."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave > orig / lo:
                f = f / fac
            elif wave >= orig / hi:
                s = (orig / wave - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_pairs(x, positions, freqs):
    """Rotation of neighbouring pairs (2i, 2i + 1) of the first 2 len(freqs) entries of the last axis by the
    angle position * freqs[i]; the rest passes.  x [T, ..., n], positions [T]."""
    T, half = x.shape[0], freqs.shape[0]
    dims = 2 * half
    out = x.clone()
    a = positions.to(F64)[:, None] * freqs[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def short_convolution(u, taps):
    """y_t[c] = sum_j taps[c, j] u_(t - K + 1 + j)[c] with zeros before the first row; u [T, C], taps [C, K]."""
    T, C = u.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=u.dtype), u])
    y = torch.zeros_like(u)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j][None, :]
    return y


# ------------------------------------------------------------------------------ mixers
def biased_talking_attention(n, W, m, rnd=_same):
    """Grouped causal attention with biases on q, k, v; the score of query i and key j is
    q.k * scale - r1_h ln(1 + r2_h (i - j)); after the softmax the heads' weights are mixed,
    p'_h = sum_g talk[h, g] p_g, and head h applies p'_h to the values of its own kv head; the head's output is
    gated by sigmoid(W_g n)_h."""
    T = n.shape[0]
    H, G, dk, dv, scale = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"]
    q = rnd(n @ W["q"].T + W["q.b"]).view(T, H, dk)
    k = rnd(n @ W["k"].T + W["k.b"]).view(T, G, dk)
    v = rnd(n @ W["v"].T + W["v.b"]).view(T, G, dv)
    gate = torch.sigmoid(n @ W["g"].T)                                  # [T, H]
    i = torch.arange(T)
    dist = (i[:, None] - i[None, :]).clamp_min(0).to(F64)
    causal = i[:, None] >= i[None, :]
    p = torch.zeros(H, T, T, dtype=n.dtype)
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale - W["r1"][h] * torch.log1p(W["r2"][h] * dist)
        p[h] = torch.softmax(s.masked_fill(~causal, -math.inf), -1)
    mixed = torch.einsum("hg,gij->hij", W["talk"], p)
    out = torch.zeros(T, H, dv, dtype=n.dtype)
    for h in range(H):
        out[:, h] = (rnd(mixed[h]) @ v[:, h // (H // G)]) * gate[:, h:h + 1]
    return rnd(out.reshape(T, H * dv)) @ W["o"].T


def forget_gate_recurrence(n, W, m, eps, rnd=_same, state=None):
    """Per head a state S [dim, vdim], zero at the start: f = lower + (1 - lower) sigmoid(W_f n + b) per key
    channel; S <- diag(f) S + (1 - f) v^T; o = S^T silu(W_q n).  Each head's o is normed over vdim with one weight
    for all heads, then W_o.  Returns (output, final state)."""
    T = n.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = rnd(torch.nn.functional.silu(n @ W["q"].T)).view(T, H, dk)
    v = rnd(n @ W["v"].T).view(T, H, dv)
    lower = W["lower"].view(H, dk)
    f = lower + (1.0 - lower) * torch.sigmoid(rnd(n @ W["f"].T + W["f.b"]).view(T, H, dk))
    S = torch.zeros(H, dk, dv, dtype=n.dtype) if state is None else state.clone()
    o = torch.zeros(T, H, dv, dtype=n.dtype)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = plain_norm(o, W["norm"], eps)
    return rnd(o.reshape(T, H * dv)) @ W["o"].T, S


def pair_mixer(n, W, m, eps, rnd=_same):
    """Two mixers on the same input; each output is normed over the width with its own plain weight, and the
    result is half their sum."""
    left = biased_talking_attention(n, {k[5:]: t for k, t in W.items() if k.startswith("left.") and k != "left.out"}, m["left"], rnd)
    right, _ = forget_gate_recurrence(n, {k[6:]: t for k, t in W.items() if k.startswith("right.") and k != "right.out"}, m["right"], eps, rnd)
    return 0.5 * (plain_norm(left, W["left.out"], eps) + plain_norm(right, W["right.out"], eps))


def conv_rotary_attention(n, W, m, eps, rnd=_same):
    """Grouped causal attention: q, k, v each pass a short causal convolution per channel right after their
    projection; q and k are normed per head (one weight for all heads) and then rotated over their first rot.dims
    channels; the head's output is gated by sigmoid(W_g n)_h."""
    T = n.shape[0]
    H, G, dk, dv, scale = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"]
    pos = torch.arange(T)
    conv = lambda u, name: rnd(short_convolution(u, W[name])) if name in W else u          # (no taps: as projected)
    q = conv(rnd(n @ W["q"].T), "q.conv").view(T, H, dk)
    k = conv(rnd(n @ W["k"].T), "k.conv").view(T, G, dk)
    v = conv(rnd(n @ W["v"].T), "v.conv").view(T, G, dv)
    q, k = plain_norm(q, W["q.norm"], eps), plain_norm(k, W["k.norm"], eps)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        fr = scaled_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
        q, k = rotate_pairs(q, pos, fr), rotate_pairs(k, pos, fr)
    q, k = rnd(q), rnd(k)
    gate = torch.sigmoid(n @ W["g"].T)
    causal = pos[:, None] >= pos[None, :]
    out = torch.zeros(T, H, dv, dtype=n.dtype)
    for h in range(H):
        g = h // (H // G)
        s = ((q[:, h] @ k[:, g].T) * scale).masked_fill(~causal, -math.inf)
        out[:, h] = (rnd(torch.softmax(s, -1)) @ v[:, g]) * gate[:, h:h + 1]
    return rnd(out.reshape(T, H * dv)) @ W["o"].T


# ------------------------------------------------------------------------ feed-forward
def squared_relu_mlp(n, W, rnd=_same):
    a = torch.relu(n @ W["up"].T + W["up.b"])
    return rnd(a * a) @ W["down"].T + W["down.b"]


# ------------------------------------------------------------------------------- model
def run_order(cfg: dict) -> list:
    """[(layer, first of a later pass)] in the order the layers run."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, times = lp["start"], lp["stop"], lp["times"]
    out = [(i, False) for i in range(a)]
    for p in range(times):
        out += [(i, p > 0 and i == a) for i in range(a, b)]
    return out + [(i, False) for i in range(b, n)]


def _sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: dict, tokens, rnd=_same, layers_out=None) -> torch.Tensor:
    """float64 logits [T, vocab] of one sequence.  layers_out: a list that receives the residual stream after
    every layer run."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    x = x0.clone()
    for i, again in run_order(cfg):
        layer, L = cfg["layers"][i], _sub(W, f"l{i}.")
        if again:
            x = x + x0
        n = rnd(offset_norm(x, L["norm1"], eps))
        if layer["type"] == "parallel":
            y = pair_mixer(n, _sub(L, "mix."), layer["mixer"], eps, rnd)
        elif layer["type"] == "attention":
            y = conv_rotary_attention(n, _sub(L, "mix."), layer["mixer"], eps, rnd)
        else:
            raise ValueError(layer["type"])
        x = x + mult * offset_norm(y, L["norm1b"], eps)
        if layer.get("mlp") is not None:
            n = rnd(offset_norm(x, L["norm2"], eps))
            x = x + mult * offset_norm(squared_relu_mlp(n, _sub(L, "mlp."), rnd), L["norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rnd(offset_norm(x, W["final.norm"], eps)) @ W["head"].T


def greedy(cfg: dict, weights: dict, prompt, n_new: int) -> list:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(cfg, weights, toks)[-1])))
    return toks[len(prompt):]
