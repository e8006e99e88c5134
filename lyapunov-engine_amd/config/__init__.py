from .engine_config import EngineConfig, parse_dtype
from .faledra_config import FaledraConfig
from .model_config import ConfigError, LlamaConfig, RopeScaling
from .ronupel_config import RonupelConfig
from .tonilix_config import TonilixConfig
from .vobotar_config import VobotarConfig
from .registry import (ARCHITECTURES, BLOCKS, EMBEDDINGS, FEED_FORWARDS, FILTERS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS,
                       STREAM_SHIFTS,
                       Architecture, Registry, architecture_of, load_config, register_architecture)
from .specs import HF_LAYER_NAMES, HF_PREFIXES, LayerCall, LayerSpec, ModelSpec, PartSpec, default_schedule

__all__ = [
    "EngineConfig", "parse_dtype", "ConfigError", "FaledraConfig", "RonupelConfig", "TonilixConfig", "VobotarConfig", "LlamaConfig", "RopeScaling", "ARCHITECTURES", "BLOCKS",
    "EMBEDDINGS", "HEADS", "FILTERS", "STREAM_SHIFTS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Architecture", "Registry", "architecture_of",
    "load_config", "register_architecture", "LayerCall", "LayerSpec", "ModelSpec", "PartSpec", "default_schedule",
    "HF_LAYER_NAMES", "HF_PREFIXES",
]
