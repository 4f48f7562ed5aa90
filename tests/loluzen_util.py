"""Helpers of the Loluzen tests: small configurations, weights that make every mechanism loud, folders."""
from __future__ import annotations

import json
import math
import os

import torch


def pair(left, right):
    """left (heads, kv_heads, dim, vdim, scale), right (heads, dim, vdim)."""
    return {"type": "parallel", "mixer": {"left": dict(zip(("heads", "kv_heads", "dim", "vdim", "scale"), left)),
                                          "right": dict(zip(("heads", "dim", "vdim"), right))}}


def attn(heads, kv_heads, dim, vdim, scale, conv=None, rot=None, base=10000.0, scaling=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if conv is not None:
        m["conv"] = conv
    if rot is not None:
        m["rot"] = {"base": base, "dims": rot}
        if scaling is not None:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": m}


def layer(mixer: dict, ff=None) -> dict:
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


def config(width, vocab, layers, loop=None, eps=1e-5, mult=0.5, scale=2.0) -> dict:
    out = {"architecture": "Loluzen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
           "residual_mult": mult, "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# Configurations that differ in every size and option: values as wide as keys and not, grouped heads, one head and a kv
# head a query head, two to five taps, one tap (a factor a channel, no state) and no convolution, all, some and none of
# a head's channels turning, scaled frequencies whose three ranges are all hit and none, key sizes of the recurrence on
# both sides of 32, a looped stretch in the middle, at the start, of one pass and none, layers without a feed-forward,
# widths that are no multiples of 8, multipliers and scales of 1 and not.
L_MIXED = config(64, 211, [
    layer(pair((4, 2, 16, 16, 0.3), (2, 16, 24)), 40),
    layer(attn(4, 2, 24, 16, 0.25, conv=3, rot=8, base=500.0, scaling=(4.0, 1.0, 4.0, 64)), 48),
    layer(pair((2, 1, 32, 8, 0.2), (3, 8, 16))),
    layer(attn(2, 2, 16, 16, 0.3, conv=2, rot=16), 24),
], loop=(1, 3, 2), mult=0.4, scale=3.0)
L_WIDE = config(96, 333, [
    layer(attn(2, 1, 64, 64, 0.125, conv=4, rot=64, base=10000.0, scaling=(8.0, 1.0, 4.0, 256)), 64),
    layer(pair((6, 3, 40, 40, 0.15), (4, 64, 32)), 72),
    layer(attn(3, 3, 40, 24, 0.16, conv=5, rot=20, base=100.0), None),
], loop=(0, 2, 3), mult=0.3, scale=8.0)
L_ODD = config(52, 97, [
    layer(pair((1, 1, 20, 12, 0.25), (1, 12, 20)), 30),
    layer(attn(5, 5, 12, 20, 0.3, conv=1, rot=2, base=7.0), None),
    layer(attn(2, 1, 8, 8, 0.35), 12),
    layer(pair((3, 3, 8, 16, 0.4), (2, 40, 8)), 20),
], loop=(1, 2, 1), eps=1e-2, mult=1.0, scale=1.0)
L_PLAIN = config(48, 101, [
    layer(attn(2, 1, 24, 24, 0.2, conv=2, rot=12), 24),
    layer(pair((2, 2, 8, 24, 0.35), (2, 24, 8)), 32),
])
ONLY = {
    "pair": config(48, 101, [layer(pair((4, 2, 16, 8, 0.5), (2, 16, 24)))]),
    "pair_wide": config(64, 101, [layer(pair((8, 2, 64, 64, 0.125), (2, 96, 16)))]),
    "attention": config(48, 101, [layer(attn(4, 2, 24, 8, 0.4, conv=4, rot=12, scaling=(4.0, 1.0, 2.0, 32)))]),
    "attention_equal": config(64, 101, [layer(attn(4, 1, 64, 64, 0.25, conv=3, rot=32))]),
    "attention_bare": config(48, 101, [layer(attn(2, 2, 24, 24, 0.4))]),
    "mlp": config(40, 101, [layer(attn(1, 1, 8, 8, 0.3), 20)]),
    "loop": config(40, 101, [layer(attn(1, 1, 8, 8, 0.3, conv=2), 16), layer(pair((1, 1, 8, 8, 0.3), (1, 8, 8)))], loop=(0, 2, 3), scale=5.0),
}
CONFIGS = dict(mixed=L_MIXED, wide=L_WIDE, odd=L_ODD, plain=L_PLAIN, **{"only_" + k: v for k, v in ONLY.items()})


def make_weights(raw: dict, seed: int, peaky: float = 1.0) -> dict:
    """bfloat16 tensors for a configuration, scaled so that every mechanism moves the logits: the mixers' outputs are far
    from zero, forget gates spread over (0, 1), distance penalties and the heads' mixing matrix are far from nothing,
    gates are not all half open, biases are not small, norm weights spread.  peaky: a factor on W_q and W_k of the
    attention mixers, so that single keys hold the weight."""
    from tuff_amd.models.registry import build_model, config_from_dict
    g = torch.Generator().manual_seed(seed)
    model = build_model(config_from_dict(raw))
    out = {}
    for d in model.weight_decls():
        name, shape = d.name, tuple(d.shape)
        n = lambda std=1.0, mean=0.0: mean + std * torch.randn(shape, generator=g)
        parts = name.split(".")
        last = parts[-1]
        if name == "embed":
            t = n(1.0)
        elif name == "head":
            t = n(1.0 / math.sqrt(shape[1]))
        elif last in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm":
            t = n(0.2)                                           # stored around zero
        elif last in ("out", "norm"):
            t = n(0.2, 1.0)                                      # plain weights
        elif last == "lower":
            t = 0.05 + 0.9 * torch.rand(shape, generator=g)
        elif last == "r1":
            t = 0.3 + 1.5 * torch.rand(shape, generator=g)
        elif last == "r2":
            t = 0.05 + 2.0 * torch.rand(shape, generator=g)
        elif last == "talk":
            t = 0.7 * torch.eye(shape[0]) + 0.3 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = n(0.6)
        elif last == "b":
            t = n(0.5)
        elif last == "g":
            t = n(2.0 / math.sqrt(shape[1]))
        elif last == "f":
            t = n(2.5 / math.sqrt(shape[1]))
        elif last in ("q", "k") and len(shape) == 2:
            t = n(1.3 * (peaky if "right" not in parts else 1.0) / math.sqrt(shape[1]))
        elif len(shape) == 2:
            t = n(1.3 / math.sqrt(shape[1]))
        else:
            t = n(0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(raw: dict, weights: dict, out_dir: str) -> str:
    from safetensors.torch import save_file
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(out_dir, "model.safetensors"))
    return out_dir
