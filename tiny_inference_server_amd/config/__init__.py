from .model_config import (ARCHITECTURES, Architecture, ConfigError, GqaMtpConfig, config_from_dict, load_config,
                           save_config)
from .registry import Registry
from .fikevik_config import FikevikConfig
from .fipuzen_config import FipuzenConfig
from .rurorax_config import RuroraxConfig
from .fesupel_config import FesupelConfig
