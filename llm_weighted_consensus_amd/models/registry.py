"""Decoder registry: from a server model spec or a model folder to (config, model).

Two ways to name a decoder:
  * ``arch``: one of the built-in shape tables (``models.config.DECODERS``: Llama / Mistral / Mixtral), weights random
    or from a safetensors path;
  * ``model_dir``: a folder holding ``config.json`` (its "architecture" picks the class) and ``*.safetensors``.
"""
from __future__ import annotations

from pathlib import Path
from typing import Optional

import torch

from .config import (DECODERS, LimatarConfig, MadipelConfig, MerudraConfig, RerozenConfig, decoder_config,
                     load_model_config)

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def resolve_config(spec: dict):
    """The decoder config a model spec names (``model_dir`` wins over ``arch``)."""
    if spec.get("model_dir"):
        return load_model_config(spec["model_dir"])
    return decoder_config(spec["arch"])


def model_class(cfg):
    if isinstance(cfg, MadipelConfig):
        from .madipel import MadipelModel

        return MadipelModel
    if isinstance(cfg, MerudraConfig):
        from .merudra import MerudraModel

        return MerudraModel
    if isinstance(cfg, LimatarConfig):
        from .limatar import LimatarModel

        return LimatarModel
    if isinstance(cfg, RerozenConfig):
        from .rerozen import RerozenModel

        return RerozenModel
    if getattr(cfg, "num_experts", 0):
        from .mixtral import MixtralModel

        return MixtralModel
    from .llama import LlamaModel

    return LlamaModel


def load_model(model_dir: str, device="cuda", dtype=torch.bfloat16, max_position: Optional[int] = None,
               random_seed: Optional[int] = None):
    """The model of a folder (config.json + safetensors); ``random_seed``: random weights of the config's shapes
    instead of the folder's."""
    cfg = load_model_config(model_dir)
    cls = model_class(cfg)
    if dtype != torch.bfloat16 and not isinstance(cfg, (MadipelConfig, MerudraConfig, LimatarConfig, RerozenConfig)):
        raise ValueError(f"{cfg.name}: this decoder runs in bfloat16 only")
    path = None if random_seed is not None else str(Path(model_dir))
    return cls(cfg, device=device, dtype=dtype, seed=random_seed or 0, weights_path=path, max_position=max_position)


__all__ = ["DECODERS", "DTYPES", "load_model", "model_class", "resolve_config"]
