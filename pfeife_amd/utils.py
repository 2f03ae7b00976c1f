"""Small host helpers shared by the front-end (logger, device moves, seeding).

Counterparts in the reference: pfeife/utils.py:14-39 (logger, to_device),
:87-96 (list_params), :209-216 (set_seed)."""
import logging
import random

import torch
from torch.utils._pytree import tree_map

_LOGGER_NAME = "pfeife"


def get_logger():
    logger = logging.getLogger(_LOGGER_NAME)
    if not logger.handlers:
        handler = logging.StreamHandler()
        handler.setFormatter(logging.Formatter("[%(levelname)s] %(message)s"))
        logger.addHandler(handler)
        logger.setLevel(logging.INFO)
        logger.propagate = False
    return logger


def set_logger_level(level):
    get_logger().setLevel(level)


def fmem(nbytes):
    """Human readable MiB string used in memory reports."""
    return "%.2fMB" % (nbytes / (1024.0 * 1024.0))


def to_device(value, device):
    """Move every tensor inside a pytree to `device`; other leaves pass through."""

    def move(v):
        return v.to(device) if torch.is_tensor(v) else v

    return tree_map(move, value)


def list_params(module):
    return [p for p in module.parameters()]


def set_seed(seed):
    random.seed(seed)
    torch.manual_seed(seed)
    try:
        import numpy as np

        np.random.seed(seed)
    except ImportError:
        pass
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


class Recorder:
    """Running mean / standard deviation of step latencies."""

    def __init__(self):
        self.values = []

    def append(self, v):
        self.values.append(float(v))

    def mean(self):
        return sum(self.values) / len(self.values) if self.values else 0.0

    def stddev(self):
        n = len(self.values)
        if n < 2:
            return 0.0
        m = self.mean()
        return (sum((v - m) ** 2 for v in self.values) / (n - 1)) ** 0.5
