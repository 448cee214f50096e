from .llama import LlamaConfig, LlamaForCausalLM, CONFIGS as _LLAMA_CONFIGS
from .hybrid import HYBRID_CONFIGS, ReperaxConfig, ReperaxForCausalLM
from .zudisun import ZUDISUN_CONFIGS, ZudisunConfig, ZudisunForCausalLM
from .fugevik import FUGEVIK_CONFIGS, FugevikConfig, FugevikForCausalLM
from .vabedra import VABEDRA_CONFIGS, VabedraConfig, VabedraForCausalLM
from .registry import (architecture_of, build_model, load_model,
                       register_architecture)

# every family's named configs, one namespace (engine server, bench, CLI)
CONFIGS = dict(_LLAMA_CONFIGS)
CONFIGS.update(HYBRID_CONFIGS)
CONFIGS.update(ZUDISUN_CONFIGS)
CONFIGS.update(FUGEVIK_CONFIGS)
CONFIGS.update(VABEDRA_CONFIGS)

__all__ = ["LlamaConfig", "LlamaForCausalLM", "ReperaxConfig",
           "ReperaxForCausalLM", "ZudisunConfig",
           "ZudisunForCausalLM", "FugevikConfig", "FugevikForCausalLM",
           "VabedraConfig", "VabedraForCausalLM",
           "CONFIGS", "architecture_of", "build_model",
           "load_model", "register_architecture"]
