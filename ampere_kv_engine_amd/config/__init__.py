from .specs import LayerSpec, ModelSpec, PartSpec, RunEntry, default_run_order, part
from .qwen3 import ConfigError, Qwen3Config
from .registry import architecture_of, known_architectures, load_config, register_architecture
from .engine import EngineConfig

__all__ = ["LayerSpec", "ModelSpec", "PartSpec", "RunEntry", "default_run_order", "part", "ConfigError",
           "Qwen3Config", "architecture_of", "known_architectures", "load_config", "register_architecture",
           "EngineConfig"]
