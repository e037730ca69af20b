from .config import (LLAMA31_70B, LLAMA31_8B, MIXTRAL_8X7B, TINY_LLAMA, TINY_MIXTRAL, ModelConfig,
                     get_config, rope_table)

from .hybrid import HybridConfig, HybridModel, HybridWeights
from .registry import load_checkpoint, make_engine

__all__ = ["HybridConfig", "HybridModel", "HybridWeights", "load_checkpoint", "make_engine",
           "LLAMA31_70B", "LLAMA31_8B", "MIXTRAL_8X7B", "TINY_LLAMA", "TINY_MIXTRAL", "ModelConfig",
           "get_config", "rope_table"]
