"""Model families: Llama-3 (8B / 70B), Mixtral-8x7B (TP/EP-aware), Sapapel, Kivezen, Nopunex and Bibezen (single GPU)."""
from .config import PRESETS, BibezenConfig, KivezenConfig, ModelConfig, NopunexConfig, SapapelConfig, get_config
from .llama import LlamaForCausalLM


def build_model(cfg, st, dtype, device):
    if isinstance(cfg, SapapelConfig):
        from .sapapel import SapapelForCausalLM
        return SapapelForCausalLM(cfg, st, dtype, device)
    if isinstance(cfg, KivezenConfig):
        from .kivezen import KivezenForCausalLM
        return KivezenForCausalLM(cfg, st, dtype, device)
    if isinstance(cfg, NopunexConfig):
        from .nopunex import NopunexForCausalLM
        return NopunexForCausalLM(cfg, st, dtype, device)
    if isinstance(cfg, BibezenConfig):
        from .bibezen import BibezenForCausalLM
        return BibezenForCausalLM(cfg, st, dtype, device)
    if cfg.is_moe:
        from .mixtral import MixtralForCausalLM
        return MixtralForCausalLM(cfg, st, dtype, device)
    return LlamaForCausalLM(cfg, st, dtype, device)


__all__ = ["PRESETS", "ModelConfig", "SapapelConfig", "KivezenConfig", "NopunexConfig", "BibezenConfig", "get_config", "LlamaForCausalLM", "build_model"]
