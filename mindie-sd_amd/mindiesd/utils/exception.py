"""Exception types of the public API (mindiesd/utils/exception.py:16-27): the message carries the
reference's error-code prefix and is logged when the exception is built."""
from .logs import logger


class ParametersInvalid(Exception):
    def __init__(self, message):
        self.message = f"[MIE06E000001] Parameters invalid. {message}"
        logger.error(self.message)
        super().__init__(self.message)


class ConfigError(Exception):
    def __init__(self, message):
        self.message = f"[MIE06E000002] Config parameter err. {message}"
        logger.error(self.message)
        super().__init__(self.message)
