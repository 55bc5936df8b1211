"""Language-model families the LLM engine can serve, chosen by a checkpoint's
config.json: the Llama family (Hugging Face naming) and the designs with their
own naming, told apart by ``"architecture"``: the hybrid Pipizen (latent /
lightning mixers), Sodonex (chunked sigmoid attention with row state) and
Movinex (windowed softmax attention, Mamba-2 layers, a repeated stretch of
layers) and Vilulix (parallel layers; matrix memory, latent attention, windowed
attention beside a gated delta rule). A family knows how to
read its config, load or seed its weights and build its step function; the
engine, the scheduler and the command line go through this table only.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import torch

from .configs import (LlamaConfig, MovinexConfig, PipizenConfig, SodonexConfig, VilulixConfig,
                      checkpoint_config, llama_config_from_hf, movinex_config_from_json,
                      pipizen_config_from_json, sodonex_config_from_json,
                      vilulix_config_from_json)


@dataclass(frozen=True)
class Family:
    name: str
    config_cls: type
    matches: Callable[[dict], bool]
    config_from_json: Callable[[dict, str], object]
    hybrid: bool            # pages + state slots (engine/hybrid_cache.py)


def _is_pipizen(d: dict) -> bool:
    return str(d.get("architecture", "")).lower() == "pipizen"


def _is_sodonex(d: dict) -> bool:
    return str(d.get("architecture", "")).lower() == "sodonex"


def _is_movinex(d: dict) -> bool:
    return str(d.get("architecture", "")).lower() == "movinex"


def _is_vilulix(d: dict) -> bool:
    return str(d.get("architecture", "")).lower() == "vilulix"


def _is_llama(d: dict) -> bool:
    arch = " ".join(d.get("architectures") or []) + " " + str(d.get("model_type", ""))
    return "num_attention_heads" in d and ("llama" in arch.lower() or "hidden_size" in d)


FAMILIES = (
    Family("pipizen", PipizenConfig, _is_pipizen, pipizen_config_from_json, True),
    Family("sodonex", SodonexConfig, _is_sodonex, sodonex_config_from_json, True),
    Family("movinex", MovinexConfig, _is_movinex, movinex_config_from_json, True),
    Family("vilulix", VilulixConfig, _is_vilulix, vilulix_config_from_json, True),
    Family("llama", LlamaConfig, _is_llama, llama_config_from_hf, False),
)


def family_of(cfg_or_json) -> Family:
    for f in FAMILIES:
        if isinstance(cfg_or_json, dict):
            if f.matches(cfg_or_json):
                return f
        elif isinstance(cfg_or_json, f.config_cls):
            return f
    what = cfg_or_json.get("architecture", cfg_or_json.get("architectures")) \
        if isinstance(cfg_or_json, dict) else type(cfg_or_json).__name__
    raise ValueError(f"no model family serves {what!r}")


def lm_config_from_json(d: dict, name: str = "checkpoint"):
    return family_of(d).config_from_json(d, name)


def lm_config_of_checkpoint(path: str, name: str = "checkpoint"):
    d = checkpoint_config(path)
    if d is None:
        raise FileNotFoundError(f"no config.json in or beside {path}")
    return lm_config_from_json(d, name)


def load_lm_weights(cfg, path: str, device, *, dtype=torch.bfloat16, tp=None,
                    max_positions: int = 8192):
    """The checkpoint's weights in the family's device layout."""
    from . import loader
    fam = family_of(cfg)
    if fam.name == "llama":
        if dtype != torch.bfloat16:
            raise ValueError("the Llama family is served in bfloat16 only")
        return loader.load_llama(cfg, path, device, tp)
    if tp is not None and tp.world > 1:
        raise ValueError(f"{fam.name}: tensor parallel serving is not available")
    if fam.name == "sodonex":
        return loader.load_sodonex(cfg, path, device, dtype, max_positions)
    if fam.name == "movinex":
        return loader.load_movinex(cfg, path, device, dtype, max_positions)
    if fam.name == "vilulix":
        return loader.load_vilulix(cfg, path, device, dtype, max_positions)
    return loader.load_pipizen(cfg, path, device, dtype, max_positions)


def random_lm_weights(cfg, device, *, seed: int = 0, dtype=torch.bfloat16, tp=None,
                      compact: bool = False, max_positions: int = 8192):
    fam = family_of(cfg)
    if fam.name == "llama":
        from .llama import LlamaWeights
        return LlamaWeights(cfg, device, seed=seed, tp=tp, compact=compact)
    if fam.name == "sodonex":
        from .sodonex import SodonexWeights
        return SodonexWeights.random(cfg, device, seed, dtype, max_positions)
    if fam.name == "movinex":
        from .movinex import MovinexWeights
        return MovinexWeights.random(cfg, device, seed, dtype, max_positions)
    if fam.name == "vilulix":
        from .vilulix import VilulixWeights
        return VilulixWeights.random(cfg, device, seed, dtype, max_positions)
    from .pipizen import PipizenWeights
    return PipizenWeights.random(cfg, device, seed, dtype, max_positions)


def build_model(weights):
    from .llama import LlamaModel, LlamaWeights
    if isinstance(weights, LlamaWeights):
        return LlamaModel(weights)
    from .sodonex import SodonexModel, SodonexWeights
    if isinstance(weights, SodonexWeights):
        return SodonexModel(weights)
    from .movinex import MovinexModel, MovinexWeights
    if isinstance(weights, MovinexWeights):
        return MovinexModel(weights)
    from .vilulix import VilulixModel, VilulixWeights
    if isinstance(weights, VilulixWeights):
        return VilulixModel(weights)
    from .pipizen import PipizenModel
    return PipizenModel(weights)
