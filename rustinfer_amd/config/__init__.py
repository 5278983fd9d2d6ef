from .model_config import (BeloraxConfig, BeloraxLayer, ConfigError, FeedForwardSpec, GeneralDeltaSpec, LatentAttentionSpec,
                           NormedAttentionSpec, RetentionSpec, YarnScaling, LightningSpec, LlamaConfig, ModelConfig, RopeScaling,
                           TedelixConfig, TedelixLayer, WindowAttentionSpec, read_config_json,
                           GatedDeltaSpec, PilavikConfig, PilavikFeedForwardSpec, PilavikLayer, SinkLatentAttentionSpec,
                           ChannelDeltaSpec, DebuzenConfig, DebuzenLayer, GatedLinearSpec, MaskedAttentionSpec, StateSpaceSpec,
                           TwoMixerSpec)
from .registry import (ArchitectureEntry, load_model_config, register_architecture,
                       registered_architectures, resolve_architecture, unregister_architecture)
from .engine_config import EngineConfig, load_engine_config, parse_toml
