"""ctypes signatures of the dynamics / per-env-term / MLP entry points."""
from __future__ import annotations


def bind(lib) -> None:  # filled in as the entry points appear in include/ksim_hip.h
    return None
