"""One package logger; level from ``KSANA_LOGGER_LEVEL`` like ksana/utils/logger.py:27-49."""

import logging
import os

log = logging.getLogger("ksanadit_amd")
if not log.handlers:
    _h = logging.StreamHandler()
    _h.setFormatter(logging.Formatter("[%(asctime)s][%(levelname)s][ksanadit_amd] %(message)s"))
    log.addHandler(_h)
    log.setLevel(os.environ.get("KSANA_LOGGER_LEVEL", "WARNING").upper())
    log.propagate = False
