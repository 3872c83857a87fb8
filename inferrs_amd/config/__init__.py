from .spec import (AttentionSpec, EmbeddingSpec, GatedMlpSpec, HeadSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                   ScheduleEntry, SpecError, default_schedule)
from .base import ConfigError, folder_stop_ids, read_config_json
from .qwen3 import Qwen3Config
from .registry import (load_config, load_spec, register_architecture, registered_architectures,
                       resolve_architecture)
