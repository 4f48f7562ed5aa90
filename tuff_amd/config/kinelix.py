"""Configuration of the Kinelix decoder: pre-norm layers with layer norms and a learned scale per channel on
every sublayer's output; the mixers are the Mamba-2 recurrence, the gated delta rule with one decay per head and
latent attention without positions (a sink per head; a layer may read an earlier layer's latent rows); the
feed-forwards a gated dense layer or experts behind a sigmoid router whose choice is limited to groups.

config.json is nested:
    architecture: "Kinelix"      vocab, width: ints      norm: {eps}      embedding: {scale}
    logit_softcap: c (optional: logits <- c tanh(logits / c))
    layers: [{type, mixer: {...}, mlp: {...} | null}, ...]
        type "mamba2":            mixer {heads, vdim, state, groups, norm_groups, conv}
        type "delta":             mixer {heads, kv_heads, dim, vdim, conv}
        type "latent_attention":  mixer {heads, dim, vdim, kv_rank, scale, kv_from (optional: the layer whose latent rows it reads)}
        mlp {kind: "dense", ff}
        mlp {kind: "moe", router: {experts, top, scale, groups: {count, keep}}, expert: {ff}}
            (without router.groups the choice is not limited; without router.scale the weights are the plain scores)
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Optional

from .base import ConfigError, ModelConfig

MIXER_KEYS = {
    "mamba2": ("heads", "vdim", "state", "groups", "norm_groups", "conv"),
    "delta": ("heads", "kv_heads", "dim", "vdim", "conv"),
    "latent_attention": ("heads", "dim", "vdim", "kv_rank", "scale"),
}


def _is_int(v, minimum=1) -> bool:
    return isinstance(v, int) and not isinstance(v, bool) and v >= minimum


def _is_num(v) -> bool:
    return isinstance(v, (int, float)) and not isinstance(v, bool)


@dataclasses.dataclass
class KinelixConfig(ModelConfig):
    architecture: ClassVar[str] = "Kinelix"
    ignored: ClassVar[frozenset[str]] = ModelConfig.ignored | frozenset({"architecture"})

    vocab: int
    width: int
    layers: list
    embedding: dict = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-5})
    logit_softcap: Optional[float] = None
    max_positions: Optional[int] = None

    def validate(self) -> None:
        self._int("vocab")
        self._int("width")
        if not isinstance(self.embedding, dict) or not _is_num(self.embedding.get("scale")):
            raise ConfigError("embedding.scale must be a number")
        if not isinstance(self.norm, dict) or not _is_num(self.norm.get("eps")) or not self.norm["eps"] > 0:
            raise ConfigError("norm.eps must be a positive number")
        if self.logit_softcap is not None and (not _is_num(self.logit_softcap) or not self.logit_softcap > 0):
            raise ConfigError(f"logit_softcap must be a positive number, got {self.logit_softcap!r}")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_KEYS:
                raise ConfigError(f"{where}.type must be one of {sorted(MIXER_KEYS)}")
            m = layer.get("mixer")
            need = MIXER_KEYS[layer["type"]]
            lacks = [k for k in need if not isinstance(m, dict) or k not in m]
            if lacks:
                raise ConfigError(f"{where}.mixer lacks key(s): {', '.join(lacks)}")
            for k in need:
                if not (_is_num(m[k]) and m[k] > 0 if k == "scale" else _is_int(m[k])):
                    raise ConfigError(f"{where}.mixer.{k} must be a positive {'number' if k == 'scale' else 'integer'}, got {m[k]!r}")
            kind = layer["type"]
            if kind == "mamba2":
                if m["heads"] % m["groups"]:
                    raise ConfigError(f"{where}.mixer: heads {m['heads']} is no multiple of groups {m['groups']}")
                if (m["heads"] * m["vdim"]) % m["norm_groups"]:
                    raise ConfigError(f"{where}.mixer: norm_groups {m['norm_groups']} does not divide heads * vdim")
            elif kind == "delta":
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}.mixer: heads {m['heads']} is no multiple of kv_heads {m['kv_heads']}")
            else:
                src = m.get("kv_from")
                if src is not None:
                    if not _is_int(src, 0) or src >= i:
                        raise ConfigError(f"{where}.mixer.kv_from must name an earlier layer, got {src!r}")
                    other = self.layers[src]
                    if other.get("type") != "latent_attention" or other["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{where}.mixer.kv_from: layer {src} has no latent rows of its own")
                    if other["mixer"]["kv_rank"] != m["kv_rank"]:
                        raise ConfigError(f"{where}.mixer.kv_rank {m['kv_rank']} is not layer {src}'s {other['mixer']['kv_rank']}")
            self._check_mlp(layer.get("mlp"), where)

    @staticmethod
    def _check_mlp(mlp, where: str) -> None:
        if mlp is None:
            return
        if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
            raise ConfigError(f"{where}.mlp.kind must be 'dense' or 'moe' (or mlp null)")
        if mlp["kind"] == "dense":
            if not _is_int(mlp.get("ff")):
                raise ConfigError(f"{where}.mlp.ff must be a positive integer")
            return
        try:
            r = mlp["router"]
            groups = r.setdefault("groups", {"count": 1, "keep": 1})       # no groups named: one group of all experts, kept
            sizes = [r["experts"], r["top"], mlp["expert"]["ff"], groups["count"], groups["keep"]]
            scale = r.setdefault("scale", 1.0)
        except (KeyError, TypeError) as e:
            raise ConfigError(f"{where}.mlp lacks a key ({e})") from None
        if not all(_is_int(v) for v in sizes):
            raise ConfigError(f"{where}.mlp: sizes must be positive integers, got {sizes}")
        if not _is_num(scale):
            raise ConfigError(f"{where}.mlp.router.scale must be a number, got {scale!r}")
        E, top, _, count, keep = sizes
        if E % count or keep > count:
            raise ConfigError(f"{where}.mlp.router.groups: {count} groups of {E} experts, {keep} kept")
        if top > keep * (E // count):
            raise ConfigError(f"{where}.mlp.router: top {top} of the {keep * (E // count)} experts the kept groups hold")

    # --------------------------------------------------------------------- derived
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def to_dict(self) -> dict[str, Any]:
        out = {"architecture": self.architecture}
        out.update(dataclasses.asdict(self))
        for k in ("logit_softcap", "max_positions"):
            if out.get(k) is None:
                out.pop(k, None)
        return out
