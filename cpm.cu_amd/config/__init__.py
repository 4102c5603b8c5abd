from .base import ConfigError, ModelConfig, architecture_name, field_from, read_config_json, require
from .minicpm import MiniCPMConfig, RopeScaling, SparseConfig
