"""Model families by the ``architecture`` key of a checkpoint's ``config.json``.

The decoder-only transformer family (``ModelConfig`` / ``DecoderLM``) is the default for configs
without that key; every other family registers its config class, a random-init builder and a
checkpoint loader here, and ``get_model_config`` / ``load_model`` / the serving engine go through it.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional


@dataclass
class Family:
    config_cls: Any
    build: Callable  # (cfg, device, dtype, seed) -> model
    load: Callable  # (checkpoint dir, cfg, device, dtype) -> model


FAMILIES: Dict[str, Family] = {}


def register(architecture: str, family: Family) -> None:
    FAMILIES[architecture] = family


def family_of(config: Dict[str, Any]) -> Optional[Family]:
    return FAMILIES.get(str(config.get("architecture", "")))


def family_of_config(cfg) -> Optional[Family]:
    return FAMILIES.get(str(getattr(cfg, "architecture", "")))


def _register_builtin() -> None:
    import torch

    from . import lenitar

    def build(cfg, device=None, dtype=torch.bfloat16, seed=None):
        if seed is not None:
            torch.manual_seed(seed)
        return lenitar.LenitarLM(cfg, device=device, dtype=dtype)

    register(lenitar.ARCHITECTURE, Family(lenitar.LenitarConfig, build, lenitar.load_lenitar))

    from . import dumalix

    def build_dumalix(cfg, device=None, dtype=torch.bfloat16, seed=None):
        if seed is not None:
            torch.manual_seed(seed)
        return dumalix.DumalixLM(cfg, device=device, dtype=dtype)

    register(dumalix.ARCHITECTURE, Family(dumalix.DumalixConfig, build_dumalix, dumalix.load_dumalix))

    from . import malinex

    def build_malinex(cfg, device=None, dtype=torch.bfloat16, seed=None):
        if seed is not None:
            torch.manual_seed(seed)
        return malinex.MalinexLM(cfg, device=device, dtype=dtype)

    register(malinex.ARCHITECTURE, Family(malinex.MalinexConfig, build_malinex, malinex.load_malinex))

    from . import pamazen

    def build_pamazen(cfg, device=None, dtype=torch.bfloat16, seed=None):
        if seed is not None:
            torch.manual_seed(seed)
        return pamazen.PamazenLM(cfg, device=device, dtype=dtype)

    register(pamazen.ARCHITECTURE, Family(pamazen.PamazenConfig, build_pamazen, pamazen.load_pamazen))


_register_builtin()
