"""The Loluzen decoder put together from parts.

x = embed[token] * embedding.scale.  Every sublayer is normed before and after and joins the stream scaled:
x <- x + m * norm_b(sublayer(norm(x))), m = residual_mult, all RMS norms whose stored weight lies around zero
(x / rms * (1 + w)).  Mixers: 'parallel', two mixers side by side on the same input whose outputs are each normed
over the width (plain weights) and averaged: grouped attention with biases, no position encoding, a logarithmic
distance penalty r1_h ln(1 + r2_h (i - j)), the heads' softmax weights mixed by a learned matrix and a sigmoid gate
per head, beside a forget-gate recurrence (q = silu(W_q h), f = lower + (1 - lower) sigmoid(W_f h + b),
S <- diag(f) S + (1 - f) v^T, o = S^T q, a norm per head); and 'attention', grouped attention whose q, k and v pass a
short causal convolution, then per-head norms of q and k and a rotation of neighbouring pairs over the first
rot.dims channels with frequencies scaled by wavelength, with a sigmoid gate per head.  Feed-forward:
W_down relu(W_up h + b)^2 + b.  Layers loop.start .. loop.stop - 1 run loop.times times in a row on the same tensors,
each pass with cache and state of its own; before every pass but the first the scaled embedding joins the stream
again.  Logits = head norm(x).

Tensors: 'embed', 'head', 'final.norm'; layer i: 'l<i>.norm1', 'l<i>.norm1b', 'l<i>.norm2', 'l<i>.norm2b',
'l<i>.mix.*' ('left.*', 'right.*', 'left.out', 'right.out' in a parallel layer), 'l<i>.mlp.up|up.b|down|down.b'.
"""
from __future__ import annotations

from ..config.loluzen import LoluzenConfig
from ..parts.attention import AttentionMixer
from ..parts.base import WeightDecl
from ..parts.block import SandwichBlock
from ..parts.ffn import DenseMLP
from ..parts.norm import RMSNorm
from ..parts.pair import PairMixer
from ..parts.recurrent import ForgetGateMixer
from ..parts.rope import Rotary
from .decoder import DecoderModel, LayerRun

ROTARY_TABLE_POSITIONS = 8192          # cosines and sines of this many positions are kept in a table


def _norm(cfg: LoluzenConfig, name: str) -> RMSNorm:
    return RMSNorm(cfg.width, cfg.eps, name, offset=1.0)


def _mixer(cfg: LoluzenConfig, i: int):
    layer, d, p = cfg.layers[i], cfg.width, f"l{i}.mix."
    m = layer["mixer"]
    if layer["type"] == "parallel":
        a, r = m["left"], m["right"]
        lp, rp = p + "left.", p + "right."
        left = AttentionMixer(d, a["heads"], a["kv_heads"], a["dim"], value_dim=a["vdim"], scale=a["scale"], exact_weights=True,
                              names={k: lp + k for k in ("q", "k", "v", "o", "q.b", "k.b", "v.b", "r1", "r2", "talk", "g")})
        right = ForgetGateMixer(d, r["heads"], r["dim"], r["vdim"], cfg.eps,
                                names={k: rp + k for k in ("q", "f", "f.b", "lower", "v", "norm", "o")})
        return PairMixer(d, left, right, cfg.eps, names={"left_norm": lp + "out", "right_norm": rp + "out"}, coef=0.5)
    rot = m.get("rot")
    position = None
    if rot and rot["dims"]:
        position = Rotary(m["dim"], rot["base"], rotary_dim=rot["dims"], interleaved=True, scaling=rot.get("scaling"),
                          table_positions=ROTARY_TABLE_POSITIONS)
    names = {k: p + k for k in ("q", "k", "v", "o", "g", "q.conv", "k.conv", "v.conv")}
    names.update(q_norm=p + "q.norm", k_norm=p + "k.norm")
    taps = m.get("conv")
    if taps is None:
        for k in ("q.conv", "k.conv", "v.conv"):
            names.pop(k)
    return AttentionMixer(d, m["heads"], m["kv_heads"], m["dim"], value_dim=m["vdim"], scale=m["scale"],
                          qk_norm_eps=cfg.eps, position=position, conv_taps=taps, names=names, exact_weights=True)


def _feed_forward(cfg: LoluzenConfig, i: int):
    spec, p = cfg.layers[i].get("mlp"), f"l{i}.mlp."
    if spec is None:
        return None
    return DenseMLP(cfg.width, spec["ff"], activation="relu2", bias=True, names={k: p + k for k in ("up", "up.b", "down", "down.b")})


def build_loluzen(cfg: LoluzenConfig) -> DecoderModel:
    d = cfg.width
    blocks = []
    for i in range(len(cfg.layers)):
        ffn = _feed_forward(cfg, i)
        before2 = _norm(cfg, f"l{i}.norm2") if ffn is not None else None
        after2 = _norm(cfg, f"l{i}.norm2b") if ffn is not None else None
        blocks.append(SandwichBlock(_norm(cfg, f"l{i}.norm1"), _mixer(cfg, i), _norm(cfg, f"l{i}.norm1b"), before2, ffn, after2,
                                    mult=cfg.residual_mult))
    runs = [LayerRun(i, reinject=again) for i, again in cfg.run_order()]       # every run has cache and state of its own
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=d, embedding=WeightDecl("embed", (cfg.vocab, d), "normal"),
        blocks=blocks, final_norm=_norm(cfg, "final.norm"), head=WeightDecl("head", (cfg.vocab, d), "normal"),
        schedule=runs, max_positions=cfg.max_positions, embedding_scale=cfg.embedding_scale, pad_hidden=True)
