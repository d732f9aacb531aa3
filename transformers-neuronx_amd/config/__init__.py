from .model_config import REQUIRED, ConfigError, ModelConfig
from .engine_config import (ContinuousBatchingConfig, EngineConfig, GenerationConfig,
                            NeuronConfig, parse_dtype)
from .registry import (Architecture, add_architecture_package, known_architectures, read_config,
                       register_architecture, resolve)
