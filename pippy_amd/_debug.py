"""Logging level of the package from the environment (reference ``pippy/_debug.py:8-21``).

``PIPPY_VERBOSITY`` = WARNING (default), INFO or DEBUG sets the level of the ``pippy_amd`` logger,
under which every module of the package logs (per-action lines of the schedules and stages at
DEBUG).  An unknown value falls back to WARNING with a warning.
"""
import logging
import os

import torch

_LEVELS = ("WARNING", "INFO", "DEBUG")


def configure(value=None) -> str:
    level = value if value is not None else os.getenv("PIPPY_VERBOSITY", "WARNING")
    if level not in _LEVELS:
        logging.warning(f"Unsupported PIPPY_VERBOSITY level: {level}")
        level = "WARNING"
    logging.getLogger("pippy_amd").setLevel(level)
    return level


PIPPY_VERBOSITY = configure()


def friendly_debug_info(v):
    """Shape and grad flag of a tensor, ``str`` of anything else."""
    if isinstance(v, torch.Tensor):
        return f"Tensor({tuple(v.shape)}, grad={v.requires_grad})"
    return str(v)


def map_debug_info(a):
    """``friendly_debug_info`` over the leaves of a list / tuple / dict."""
    return torch.fx.node.map_aggregate(a, friendly_debug_info)
