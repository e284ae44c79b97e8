from .base import ConfigError, KeyReader, read_config_json
from .specs import (NormSpec, PositionSpec, MixerSpec, FeedForwardSpec, LayerSpec, EmbeddingSpec, HeadSpec,
                    CacheNeed, ScheduleEntry, ModelSpec, params)
from .llama import LlamaConfig, RopeScaling
from .registry import (register_architecture, lookup_architecture, architecture_of,
                       architecture_names, config_from_dict, config_from_folder, model_spec_of)
