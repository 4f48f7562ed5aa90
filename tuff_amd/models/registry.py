"""One table from an architecture's name (config.json `architectures[0]`) to its configuration
class and the function that builds its model.  The reference keeps the same table as an enum
plus a switch over engine vtables (include/tuff_vtable.h:13-57, src/tuff_vtable.c:159-171).
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Type

from ..config.base import ConfigError, ModelConfig, architecture_name, read_config_json


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Type[ModelConfig]
    build: Callable[[ModelConfig], "object"]      # -> DecoderModel


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], build: Callable) -> None:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_cls, build)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def get_architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture '{name}'; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def config_from_dict(raw: dict) -> ModelConfig:
    return get_architecture(architecture_name(raw)).config_cls.from_dict(raw)


def load_config(model_dir: str) -> ModelConfig:
    """The folder's configuration.  A configuration that leaves sizes to the tensors' shapes (it has a
    with_shapes method) is completed from the checkpoint's headers; no tensor is read for it."""
    cfg = config_from_dict(read_config_json(model_dir))
    if hasattr(cfg, "with_shapes"):
        from ..weights.loader import Checkpoint
        from ..weights.safetensors_io import SafetensorsError
        try:
            ck = Checkpoint(model_dir)
        except (SafetensorsError, OSError):
            return cfg                    # no readable checkpoint: the loader says so when the weights are asked for
        names = set(ck.names())
        cfg = cfg.with_shapes(lambda n: ck.shape(n) if n in names else None)
    return cfg


def build_model(cfg: ModelConfig):
    return get_architecture(cfg.architecture).build(cfg)


def _register_builtin() -> None:
    from ..config.lfm2 import Lfm2Config
    from .lfm2 import build_lfm2
    register_architecture(Lfm2Config.architecture, Lfm2Config, build_lfm2)
    from ..config.pafodra import PafodraConfig
    from .pafodra import build_pafodra
    register_architecture(PafodraConfig.architecture, PafodraConfig, build_pafodra)
    from ..config.kugalorn import KugalornConfig
    from .kugalorn import build_kugalorn
    register_architecture(KugalornConfig.architecture, KugalornConfig, build_kugalorn)
    from ..config.loluzen import LoluzenConfig
    from .loluzen import build_loluzen
    register_architecture(LoluzenConfig.architecture, LoluzenConfig, build_loluzen)
    from ..config.kinelix import KinelixConfig
    from .kinelix import build_kinelix
    register_architecture(KinelixConfig.architecture, KinelixConfig, build_kinelix)


_register_builtin()
