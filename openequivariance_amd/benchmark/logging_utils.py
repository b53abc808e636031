"""Logger of the harness (reference: openequivariance/benchmark/logging_utils.py)."""
import logging

_logger = logging.getLogger("openequivariance_amd")
if not _logger.handlers:
    _h = logging.StreamHandler()
    _h.setFormatter(logging.Formatter("%(asctime)s %(levelname)s %(message)s"))
    _logger.addHandler(_h)
    _logger.setLevel(logging.INFO)


def getLogger():
    return _logger
