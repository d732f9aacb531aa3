from .model_config import ConfigError, ModelConfig, OPTConfig
from .engine_config import (ContinuousBatchingConfig, EngineConfig, GenerationConfig,
                            NeuronConfig, parse_dtype)
from .registry import Architecture, known_architectures, read_config, register_architecture, resolve
