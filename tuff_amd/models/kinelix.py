"""The Kinelix decoder put together from parts.

x = embed[token] * embedding.scale.  Every layer is pre-norm with layer norms (a weight, no bias) and a learned scale
per channel on each sublayer's output: x <- x + ls1 * mixer(norm1(x)), then x <- x + ls2 * ff(norm2(x)).  Mixers:
'mamba2', the state-space recurrence with a scalar decay per head behind one short convolution and a gated norm in
groups; 'delta', the gated delta rule with one decay per head and a silu output gate; 'latent_attention', latent
attention without positions whose softmax has a sink per head, and which with `kv_from` reads the latent rows that an
earlier layer keeps (its own W_uk, W_uv and queries on that layer's cache entry).  Feed-forwards: a gated dense
layer with silu, or experts of that form behind a sigmoid router whose choice runs on the scores plus a correction
and only inside the best groups of experts; the weights are the plain scores times router.scale.  Logits =
head norm(x), then softcap * tanh(logits / softcap).

Tensors: 'embed', 'head', 'final.norm'; layer i: 'l<i>.norm1', 'l<i>.norm2', 'l<i>.ls1', 'l<i>.ls2', 'l<i>.mix.*',
'l<i>.mlp.gate|up|down' or 'l<i>.mlp.e<k>.gate|up|down', 'l<i>.mlp.router', 'l<i>.mlp.correction'.
"""
from __future__ import annotations

from ..config.kinelix import KinelixConfig
from ..parts.base import WeightDecl
from ..parts.block import LayerScaleBlock
from ..parts.ffn import MoE, SwiGLU
from ..parts.latent import LatentAttentionMixer
from ..parts.norm import LayerNorm
from ..parts.recurrent import GatedDeltaMixer, Mamba2Mixer
from .decoder import DecoderModel, LayerRun


def _norm(cfg: KinelixConfig, name: str) -> LayerNorm:
    return LayerNorm(cfg.width, cfg.eps, name)


def _mixer(cfg: KinelixConfig, i: int):
    layer, d, p = cfg.layers[i], cfg.width, f"l{i}.mix."
    m = layer["mixer"]
    if layer["type"] == "mamba2":
        names = {k: p + k for k in ("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o")}
        return Mamba2Mixer(d, m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"], m["conv"], cfg.eps, names=names)
    if layer["type"] == "delta":
        names = {k: p + k for k in ("q", "k", "v", "q.conv", "k.conv", "v.conv", "b", "A_log", "a", "dt_bias", "g", "norm", "o")}
        return GatedDeltaMixer(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], cfg.eps, names=names,
                               gate_activation="silu")
    keys = ("q", "uk", "uv", "sink", "o") + (() if m.get("kv_from") is not None else ("dkv", "dkv.norm"))
    return LatentAttentionMixer(d, m["heads"], m["dim"], 0, m["vdim"], m["kv_rank"], norm_eps=cfg.eps, scale=m["scale"],
                                names={k: p + k for k in keys}, exact_weights=True)


def _feed_forward(cfg: KinelixConfig, i: int):
    spec, d, p = cfg.layers[i].get("mlp"), cfg.width, f"l{i}.mlp."
    if spec is None:
        return None
    if spec["kind"] == "dense":
        return SwiGLU(d, spec["ff"], names={k: p + k for k in ("gate", "up", "down")})
    r = spec["router"]
    names = {"router": p + "router", "correction": p + "correction",
             "experts": [(f"{p}e{k}.gate", f"{p}e{k}.up", f"{p}e{k}.down") for k in range(r["experts"])]}
    return MoE(d, r["experts"], r["top"], spec["expert"]["ff"], names=names, activation="silu", gated=True,
               router_weights="sigmoid", scale_input=False, route_groups=r["groups"]["count"], route_keep=r["groups"]["keep"],
               route_scale=float(r["scale"]))


def build_kinelix(cfg: KinelixConfig) -> DecoderModel:
    d = cfg.width
    blocks, runs = [], []
    for i, layer in enumerate(cfg.layers):
        ffn = _feed_forward(cfg, i)
        norm2 = _norm(cfg, f"l{i}.norm2") if ffn is not None else None
        names = {"ls1": f"l{i}.ls1", "ls2": f"l{i}.ls2"}
        blocks.append(LayerScaleBlock(_norm(cfg, f"l{i}.norm1"), _mixer(cfg, i), norm2, ffn, names=names))
        src = layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None
        # a layer's cache entry carries the layer's number; a reader runs on the entry of the layer it names
        runs.append(LayerRun(i, cache=i) if src is None else LayerRun(i, cache=src, writes=False))
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=d, embedding=WeightDecl("embed", (cfg.vocab, d), "normal"),
        blocks=blocks, final_norm=_norm(cfg, "final.norm"), head=WeightDecl("head", (cfg.vocab, d), "normal"),
        schedule=runs, max_positions=cfg.max_positions, embedding_scale=float(cfg.embedding["scale"]),
        logit_softcap=cfg.logit_softcap, pad_hidden=True)
