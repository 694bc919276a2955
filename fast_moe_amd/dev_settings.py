"""Developer switches of the reference package (/root/reference/dev_settings.py:14-41).

The reference uses them to pick debug paths of its Triton kernels; the HIP kernels have no such
paths, so the values are recorded and read back, nothing else depends on them.  The environment
variable FASTMOE_DEV_MODE, when set, wins over ``set_dev_mode`` as it does there.
"""
from __future__ import annotations

import logging
import os

logger = logging.getLogger(__name__)

_state = {"dev_mode": os.environ.get("FASTMOE_DEV_MODE", "0") == "1", "verbose": 0}


def set_dev_mode(val: bool) -> None:
    if "FASTMOE_DEV_MODE" in os.environ:
        logger.warning("set_dev_mode(%s) ignored: FASTMOE_DEV_MODE is set in the environment", val)
        return
    _state["dev_mode"] = bool(val)


def is_dev_mode() -> bool:
    return _state["dev_mode"]


def set_verbose_level(level: int) -> None:
    _state["verbose"] = int(level)


def get_verbose_level() -> int:
    return _state["verbose"]
