from .base import ConfigError, KeyReader, read_config_json, architecture_name
from .plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry, Source
from .registry import (Architecture, config_from_dict, config_from_dir, known_architectures,
                       lookup_architecture, register_architecture)
