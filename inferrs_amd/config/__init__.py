from .spec import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                   ScheduleEntry, SpecError, default_schedule)
from .qwen3 import ConfigError, Qwen3Config, read_config_json
from .registry import (load_config, load_spec, register_architecture, registered_architectures,
                       resolve_architecture)
