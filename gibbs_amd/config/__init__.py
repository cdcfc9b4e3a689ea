"""Typed configurations and the architecture registry."""
from .base import ArchConfig, ConfigError, first, read_config_json, require
from .lfm2 import Lfm2Config, feed_forward_width
from .zokepel import ZokepelConfig
from .rukosun import RukosunConfig
from .ruzinex import RuzinexConfig
from .litizen import LitizenConfig
from .registry import (Architecture, architectures, config_from_dict,
                       find_architecture, register_architecture)
from .spec import (ConnectionSpec, EmbeddingTablesSpec, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec,
                   PositionSpec)

register_architecture("Lfm2ForCausalLM", Lfm2Config, aliases=("lfm2",))
register_architecture("Zokepel", ZokepelConfig, aliases=("zokepel",))
register_architecture("Rukosun", RukosunConfig, aliases=("rukosun",))
register_architecture("Ruzinex", RuzinexConfig, aliases=("ruzinex",))
register_architecture("Litizen", LitizenConfig, aliases=("litizen",))
