from .exception import ParametersInvalid
from .logs import logger
from .device import is_gpu_available

__all__ = ["ParametersInvalid", "logger", "is_gpu_available"]
