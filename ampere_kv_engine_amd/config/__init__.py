from .specs import LayerSpec, ModelSpec, PartSpec, RunEntry, default_run_order, part
from .qwen3 import ConfigError, Qwen3Config
from .keranex import KeranexConfig
from .tukevik import TukevikConfig
from .lirulix import LirulixConfig
from .mekuvik import MekuvikConfig
from .registry import architecture_of, known_architectures, load_config, register_architecture
from .engine import EngineConfig

__all__ = ["LayerSpec", "ModelSpec", "PartSpec", "RunEntry", "default_run_order", "part", "ConfigError",
           "Qwen3Config", "KeranexConfig", "TukevikConfig", "LirulixConfig", "MekuvikConfig", "architecture_of", "known_architectures", "load_config", "register_architecture",
           "EngineConfig"]
