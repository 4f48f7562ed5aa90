"""Helpers of the Kinelix tests: small configurations, weights that make every mechanism loud, folders."""
from __future__ import annotations

import json
import math
import os

import torch


def mamba(heads, vdim, state, groups, norm_groups, conv):
    return {"type": "mamba2", "mixer": dict(heads=heads, vdim=vdim, state=state, groups=groups, norm_groups=norm_groups, conv=conv)}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)}


def latent(heads, dim, vdim, rank, scale, kv_from=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, kv_rank=rank, scale=scale)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, count, keep, scale):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}},
            "expert": {"ff": ff}}


def layer(mixer: dict, mlp=None) -> dict:
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, eps=1e-5, embed_scale=1.0, softcap=None) -> dict:
    out = {"architecture": "Kinelix", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": embed_scale}, "layers": layers}
    if softcap is not None:
        out["logit_softcap"] = softcap
    return out


# Configurations that differ in every size and option: one to many heads, groups of one head and of all, norms in one to
# three parts, one to five taps, keys wider and narrower than values, latent rows on and off borders of 8, a layer that
# reads another's rows (next to it and further up), one to all experts chosen, one to four groups of which one to all
# are kept, layers without a feed-forward, sizes that are no multiples of 8, scales and caps of 1 and not, no cap.
# X_MIXED chooses all its experts, so no discrete choice can turn under bfloat16 rounding and long bfloat16 runs count
# to their end; fewer than all are chosen in X_WIDE, X_ODD, X_PLAIN and the expert layers alone.
X_MIXED = config(64, 211, [
    layer(mamba(4, 8, 16, 2, 2, 4), dense(40)),
    layer(latent(2, 16, 24, 32, 0.3), moe(4, 4, 40, 2, 2, 1.5)),
    layer(delta(4, 2, 16, 8, 2), None),
    layer(latent(3, 8, 16, 32, 0.25, kv_from=1), moe(4, 4, 24, 1, 1, 0.6)),
    layer(mamba(2, 24, 8, 1, 1, 2), moe(3, 3, 16, 3, 3, 1.0)),
], embed_scale=2.0, softcap=10.0)
X_WIDE = config(96, 333, [
    layer(delta(2, 2, 40, 24, 5), moe(8, 2, 24, 4, 2, 0.7)),
    layer(mamba(6, 16, 40, 3, 1, 2), moe(6, 3, 16, 1, 1, 1.0)),
    layer(latent(4, 24, 8, 48, 0.12), dense(72)),
    layer(latent(1, 40, 40, 40, 0.1), None),
    layer(latent(5, 16, 24, 48, 0.2, kv_from=2), moe(6, 1, 40, 3, 1, 2.5)),
    layer(latent(2, 32, 16, 40, 0.15, kv_from=3), dense(24)),
], embed_scale=0.5, softcap=30.0)
X_ODD = config(52, 97, [
    layer(mamba(3, 5, 7, 1, 3, 3), moe(6, 1, 12, 3, 1, 2.0)),
    layer(latent(1, 12, 20, 20, 0.3), dense(30)),
    layer(latent(3, 5, 7, 20, 0.4, kv_from=1), None),
    layer(delta(3, 1, 10, 6, 1), moe(4, 2, 20, 2, 1, 1.0)),
], eps=1e-2)
X_PLAIN = config(48, 101, [
    layer(mamba(4, 12, 24, 4, 4, 1), dense(24)),
    layer(delta(2, 1, 24, 24, 3), moe(4, 2, 24, 2, 2, 1.2)),
    layer(latent(2, 8, 8, 16, 0.35), moe(4, 2, 24, 2, 1, 1.0)),
], softcap=1.0)
ONLY = {
    "mamba": config(48, 101, [layer(mamba(4, 8, 16, 2, 2, 4))], embed_scale=3.0),
    "mamba_one_tap": config(48, 101, [layer(mamba(2, 20, 12, 2, 1, 1))]),
    "mamba_wide_state": config(64, 101, [layer(mamba(2, 8, 72, 1, 2, 3))]),         # sixteen lanes a value channel
    # sizes the chunked form takes (multiples of 16): prompt portions of 64 tokens and more run on the matrix cores
    "mamba_sixteens": config(64, 101, [layer(mamba(4, 16, 32, 2, 1, 4)), layer(mamba(2, 48, 48, 1, 2, 2))], embed_scale=2.0),
    "delta": config(48, 101, [layer(delta(4, 2, 16, 8, 3))]),
    "delta_wide": config(64, 101, [layer(delta(2, 2, 80, 72, 2))]),
    "latent": config(48, 101, [layer(latent(2, 16, 24, 32, 0.6))]),
    "latent_wide": config(64, 101, [layer(latent(3, 24, 16, 280, 0.3))]),           # a cache row beyond the matrix-core kernels
    "latent_eights": config(48, 101, [layer(latent(8, 16, 24, 32, 0.5))]),
    "latent_many_heads": config(64, 101, [layer(latent(24, 16, 8, 152, 0.4))]),
    "latent_shared": config(48, 101, [layer(latent(2, 16, 8, 24, 0.5)), layer(latent(3, 8, 16, 24, 0.7, kv_from=0))]),
    "moe": config(48, 101, [layer(latent(1, 8, 8, 8, 0.3), moe(8, 2, 24, 4, 2, 1.5))]),
    "moe_odd": config(44, 101, [layer(latent(1, 8, 8, 8, 0.3), moe(6, 2, 20, 3, 1, 0.8))]),
    "dense": config(40, 101, [layer(latent(1, 8, 8, 8, 0.3), dense(28))], softcap=5.0),
}
CONFIGS = dict(mixed=X_MIXED, wide=X_WIDE, odd=X_ODD, plain=X_PLAIN, **{"only_" + k: v for k, v in ONLY.items()})


def make_weights(raw: dict, seed: int) -> dict:
    """bfloat16 tensors for a configuration, scaled so that every mechanism moves the logits: mixers and
    feed-forwards add about the stream's own size, the scales per channel spread around one, decays spread over
    (0, 1) with some heads remembering hundreds of tokens, sinks hold a share, the router's correction is of the
    scores' own size, the convolutions' biases are not small."""
    from tuff_amd.models.registry import build_model, config_from_dict
    g = torch.Generator().manual_seed(seed)
    model = build_model(config_from_dict(raw))
    out = {}
    for d in model.weight_decls():
        name, shape = d.name, tuple(d.shape)
        n = lambda std=1.0, mean=0.0: mean + std * torch.randn(shape, generator=g)
        last = name.split(".")[-1]
        if name == "embed":
            t = n(1.0)
        elif name == "head":
            t = n(1.0 / math.sqrt(shape[1]))
        elif last in ("ls1", "ls2"):
            t = n(0.3, 1.0)
        elif last in ("norm1", "norm2", "norm") or name == "final.norm":
            t = n(0.2, 1.0)
        elif last == "A_log":
            t = n(1.5, -1.5)                                     # rates exp(A_log) from a hundredth to one and more
        elif last == "dt_bias":
            t = n(1.0)
        elif last == "D":
            t = n(0.5, 1.0)
        elif last == "sink":
            t = n(1.0, 0.5)
        elif last == "correction":
            t = n(0.3)
        elif last == "router":
            t = n(3.0 / math.sqrt(shape[1]))
        elif last == "conv":
            t = n(0.6)
        elif name.endswith("conv.b"):
            t = n(0.3)
        elif last in ("a", "b"):
            t = n(2.0 / math.sqrt(shape[1]))
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
