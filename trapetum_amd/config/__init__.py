from .base import ConfigError, ModelConfig, key, read_config_json, architecture_name   # noqa: F401
from .gemma2 import Gemma2Config   # noqa: F401
from .golepel import GolepelConfig   # noqa: F401
from .lutovik import LutovikConfig   # noqa: F401
from .besulix import BesulixConfig   # noqa: F401
from .vogunex import VogunexConfig   # noqa: F401
