from .base import ConfigError, KeyReader, architecture_name, read_config_json
from .mistral import MistralConfig
