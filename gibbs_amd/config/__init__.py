"""Typed configurations and the architecture registry."""
from .base import ArchConfig, ConfigError, first, read_config_json, require
from .lfm2 import Lfm2Config, feed_forward_width
from .registry import (Architecture, architectures, config_from_dict,
                       find_architecture, register_architecture)
from .spec import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec,
                   PositionSpec)

register_architecture("Lfm2ForCausalLM", Lfm2Config, aliases=("lfm2",))
