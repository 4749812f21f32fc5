"""Typed configurations, the architecture registry and the neutral model description."""
from .spec import (AttentionSpec, LayerSpec, ModelSpec, RmsNormSpec, RotarySpec,
                   RunEntry, ScaleSpec, SoftCapSpec, SwiGluSpec)
from .errors import ConfigError
from .registry import (config_class_for, parse_config, read_config, register_architecture,
                       registered_architectures)
from .llama import Llama3Scaling, LlamaConfig          # registers itself
