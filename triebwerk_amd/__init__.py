"""MI355X (gfx950) KV-cache hot path of the triebwerk inference engine.

``Engine`` mirrors the reference's pybind class for this path
(engine/engine_py.cpp:21-45); ``kvcache`` exposes the kernel launchers.
"""
from .engine import Engine  # noqa: F401
from . import kvcache  # noqa: F401

__all__ = ["Engine", "kvcache"]
