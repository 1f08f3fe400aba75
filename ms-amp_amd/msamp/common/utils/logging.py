"""Package logger (stdlib logging; the reference wraps colorlog, msamp/common/utils/logging.py:34-87)."""

import logging
import socket

logger = logging.getLogger('msamp')
if not logger.handlers:
    _h = logging.StreamHandler()
    _h.setFormatter(logging.Formatter(f'[%(asctime)s {socket.gethostname()}][%(filename)s:%(lineno)s][%(levelname)s] %(message)s'))
    logger.addHandler(_h)
    logger.setLevel(logging.INFO)
    logger.propagate = False
