"""Model registry."""

from __future__ import annotations

from ..engine.config import ModelConfig


def get_model(cfg: ModelConfig):
    if cfg.architecture == "llama":
        from .llama import LlamaForCausalLM

        return LlamaForCausalLM(cfg)
    if cfg.architecture == "mixtral":
        from .mixtral import MixtralForCausalLM

        return MixtralForCausalLM(cfg)
    if cfg.architecture == "opt":
        from .opt import OPTForCausalLM

        return OPTForCausalLM(cfg)
    if cfg.architecture == "dolodra":
        from .dolodra import DolodraForCausalLM

        return DolodraForCausalLM(cfg)
    if cfg.architecture == "kezunex":
        from .kezunex import KezunexForCausalLM

        return KezunexForCausalLM(cfg)
    if cfg.architecture == "relerax":
        from .relerax import ReleraxForCausalLM

        return ReleraxForCausalLM(cfg)
    if cfg.architecture == "gumozen":
        from .gumozen import GumozenForCausalLM

        return GumozenForCausalLM(cfg)
    raise ValueError(f"Unsupported architecture: {cfg.architecture}")


def native_extensions(cfg: ModelConfig) -> list[str]:
    """Names of the compiled extensions (kernels/build.py) whose ops the
    model's forward reaches on a GPU — what a fresh checkout has to build
    before it can serve this model."""
    if cfg.architecture == "dolodra":
        return ["_C_seq", "_C_lat"]
    if cfg.architecture == "kezunex":
        from .kezunex import native_extensions as kz

        return kz(cfg)
    if cfg.architecture == "relerax":
        from .relerax import native_extensions as rx

        return rx(cfg)
    if cfg.architecture == "gumozen":
        from .gumozen import native_extensions as gz

        return gz(cfg)
    return ["_C"]
