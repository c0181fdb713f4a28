from .model_config import ConfigError, Qwen3Config, architecture_name, read_config_json
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
