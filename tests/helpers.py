"""Shared helpers for the tests: package loading and seeded inputs."""
import os
import re
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from __graft_entry__ import load_package  # noqa: E402

HEADER = os.path.join(ROOT, "include", "itak_hip_kv.h")


def pkg():
    return load_package()


def declared_symbols():
    """Function names declared in include/itak_hip_kv.h."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(itak_[a-z0-9_]+)\s*\(", text)))


def normal(rng, *shape):
    return rng.standard_normal(shape, dtype=np.float32)


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64))))


def rel_err(a, b):
    """Max abs difference relative to the largest magnitude of the reference tensor."""
    return max_abs(a, b) / float(np.max(np.abs(b)))
