from .llama import LlamaConfig, LlamaForCausalLM, CONFIGS as _LLAMA_CONFIGS
from .hybrid import HYBRID_CONFIGS, ReperaxConfig, ReperaxForCausalLM
from .registry import (architecture_of, build_model, load_model,
                       register_architecture)

# every family's named configs, one namespace (engine server, bench, CLI)
CONFIGS = dict(_LLAMA_CONFIGS)
CONFIGS.update(HYBRID_CONFIGS)

__all__ = ["LlamaConfig", "LlamaForCausalLM", "ReperaxConfig",
           "ReperaxForCausalLM", "CONFIGS", "architecture_of", "build_model",
           "load_model", "register_architecture"]
