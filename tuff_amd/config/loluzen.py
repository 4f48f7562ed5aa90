"""Configuration of the Loluzen decoder: layers whose sublayers are normed before and after
(x <- x + m * norm_after(sublayer(norm_before(x)))), each with a pair of mixers side by side or an
attention mixer behind short convolutions, and a dense feed-forward or none; a stretch of the layers
may run several times in a row, the scaled embedding joining the stream again before every later pass.

config.json is nested:
    architecture: "Loluzen"     vocab, width: ints     norm: {eps}     embedding: {scale}     residual_mult: m
    loop: {start, stop, times} (optional: layers start .. stop - 1 run `times` times in a row)
    layers: [{type, mixer: {...}, mlp: {...} | null}, ...]
        type "parallel":   mixer {left: {heads, kv_heads, dim, vdim, scale}, right: {heads, dim, vdim}}
        type "attention":  mixer {heads, kv_heads, dim, vdim, scale, conv: taps,
                                  rot: {base, dims, scaling: {factor, low, high, original} (optional)}}
        mlp {kind: "dense", ff}
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Optional

from .base import ConfigError, ModelConfig

ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
RECURRENT_KEYS = ("heads", "dim", "vdim")
SCALING_KEYS = ("factor", "low", "high", "original")


def _is_int(v, minimum=1) -> bool:
    return isinstance(v, int) and not isinstance(v, bool) and v >= minimum


def _is_pos(v) -> bool:
    return isinstance(v, (int, float)) and not isinstance(v, bool) and v > 0


def _check_sizes(where: str, m, keys) -> None:
    lacks = [k for k in keys if not isinstance(m, dict) or k not in m]
    if lacks:
        raise ConfigError(f"{where} lacks key(s): {', '.join(lacks)}")
    for k in keys:
        if not (_is_pos(m[k]) if k == "scale" else _is_int(m[k])):
            raise ConfigError(f"{where}.{k} must be a positive {'number' if k == 'scale' else 'integer'}, got {m[k]!r}")
    if "kv_heads" in keys and m["heads"] % m["kv_heads"]:
        raise ConfigError(f"{where}: heads {m['heads']} is no multiple of kv_heads {m['kv_heads']}")


@dataclasses.dataclass
class LoluzenConfig(ModelConfig):
    architecture: ClassVar[str] = "Loluzen"
    ignored: ClassVar[frozenset[str]] = ModelConfig.ignored | frozenset({"architecture"})

    vocab: int
    width: int
    layers: list
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    embedding: dict = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    residual_mult: float = 1.0
    loop: Optional[dict] = None
    max_positions: Optional[int] = None

    def validate(self) -> None:
        self._int("vocab")
        self._int("width")
        self._float("residual_mult", positive=False)
        if not isinstance(self.norm, dict) or not _is_pos(self.norm.get("eps")):
            raise ConfigError("norm.eps must be a positive number")
        if not isinstance(self.embedding, dict) or not isinstance(self.embedding.get("scale"), (int, float)) \
                or isinstance(self.embedding.get("scale"), bool):
            raise ConfigError("embedding.scale must be a number")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in ("parallel", "attention"):
                raise ConfigError(f"{where}.type must be 'parallel' or 'attention'")
            m = layer.get("mixer")
            if layer["type"] == "parallel":
                if not isinstance(m, dict):
                    raise ConfigError(f"{where}.mixer must give left and right")
                _check_sizes(f"{where}.mixer.left", m.get("left"), ATTENTION_KEYS)
                _check_sizes(f"{where}.mixer.right", m.get("right"), RECURRENT_KEYS)
            else:
                _check_sizes(f"{where}.mixer", m, ATTENTION_KEYS)
                if m.get("conv") is not None and not _is_int(m["conv"]):
                    raise ConfigError(f"{where}.mixer.conv must be a positive number of taps, got {m.get('conv')!r}")
                rot = m.get("rot")
                if rot is not None:
                    if not isinstance(rot, dict) or not _is_pos(rot.get("base")) or not _is_int(rot.get("dims"), 0):
                        raise ConfigError(f"{where}.mixer.rot must give base and dims")
                    if rot["dims"] % 2 or rot["dims"] > m["dim"]:
                        raise ConfigError(f"{where}.mixer.rot.dims must be even and at most dim, got {rot['dims']}")
                    sc = rot.get("scaling")
                    if sc is not None:
                        if not isinstance(sc, dict) or not all(_is_pos(sc.get(k)) for k in SCALING_KEYS):
                            raise ConfigError(f"{where}.mixer.rot.scaling must give positive {', '.join(SCALING_KEYS)}")
                        if not sc["high"] > sc["low"]:
                            raise ConfigError(f"{where}.mixer.rot.scaling: high must lie above low")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp.kind must be 'dense' (or mlp null)")
                if not _is_int(mlp.get("ff")):
                    raise ConfigError(f"{where}.mlp.ff must be a positive integer, got {mlp.get('ff')!r}")
        if self.loop is not None:
            lp = self.loop
            ok = isinstance(lp, dict) and all(_is_int(lp.get(k), 0) for k in ("start", "stop")) and _is_int(lp.get("times"))
            if not ok or not 0 <= lp["start"] <= lp["stop"] <= len(self.layers):
                raise ConfigError(f"loop must give 0 <= start <= stop <= {len(self.layers)} and times >= 1, got {lp!r}")

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

    @property
    def embedding_scale(self) -> float:
        return float(self.embedding["scale"])

    def run_order(self) -> list[tuple]:
        """[(layer, the embedding joins the stream before it)] in the order the layers run: the looped stretch
        `times` times in a row, and the first layer of every pass after the first takes the embedding again."""
        n = len(self.layers)
        if not self.loop:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        out = [(i, False) for i in range(a)]
        for p in range(times):
            out += [(i, p > 0 and i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    def to_dict(self) -> dict[str, Any]:
        out = {"architecture": self.architecture}
        out.update(dataclasses.asdict(self))
        for k in ("loop", "max_positions"):
            if out.get(k) is None:
                out.pop(k, None)
        return out
