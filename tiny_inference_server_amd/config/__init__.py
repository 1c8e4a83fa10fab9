from .model_config import (ARCHITECTURES, Architecture, ConfigError, GqaMtpConfig, config_from_dict, load_config,
                           save_config)
from .registry import Registry
