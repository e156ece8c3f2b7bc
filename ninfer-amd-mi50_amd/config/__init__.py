from .base import ConfigError, KeyReader, architecture_name, read_config_json
from .fopinex import FopinexConfig
from .getodra import GetodraConfig
from .options import EngineOptions
from .qwen2_moe import Qwen2MoeConfig
from .sosepel import SosepelConfig
from .tuzapel import TuzapelConfig

__all__ = ["ConfigError", "KeyReader", "architecture_name", "read_config_json",
           "EngineOptions", "FopinexConfig", "GetodraConfig", "Qwen2MoeConfig", "SosepelConfig", "TuzapelConfig"]
