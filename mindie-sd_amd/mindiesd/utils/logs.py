"""Package logger.  Same logger name as the reference (``'mindie-sd'``,
mindiesd/utils/logs/logging.py:347-398); level from ``MINDIE_LOG_LEVEL`` (default: warning).
Unlike the reference no log file is created on import."""
import logging
import os

logger = logging.getLogger("mindie-sd")
if not logger.handlers:
    _h = logging.StreamHandler()
    _h.setFormatter(logging.Formatter("[%(asctime)s] [%(levelname)s] [mindie-sd] %(message)s"))
    logger.addHandler(_h)
    logger.propagate = False
logger.setLevel(getattr(logging, os.getenv("MINDIE_LOG_LEVEL", "WARNING").upper(), logging.WARNING))
