from .exception import ConfigError, ParametersInvalid
from .logs import logger
from .device import is_gpu_available

__all__ = ["ConfigError", "ParametersInvalid", "logger", "is_gpu_available"]
