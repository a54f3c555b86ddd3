"""Eager / graph-capturing mode flag read by the linear dispatcher.

Mirrors the part of the reference's ``phyai/parallel/state.py:20-44`` that the
linear path touches: a ``Mode`` enum, ``current_mode()`` and the
``graph_capture()`` context manager that the graph wrapper enters around
capture.  Kernel selection is cached per mode, so a kernel that cannot be
recorded into a graph is never picked while one is being captured.  The mesh
registry of the reference module is not reproduced: this build is single-GPU.
"""

from __future__ import annotations

import contextlib
import contextvars
import enum


class Mode(enum.Enum):
    EAGER = "eager"
    GRAPH_CAPTURING = "graph_capturing"


_MODE: contextvars.ContextVar[Mode] = contextvars.ContextVar("phyai_amd_mode", default=Mode.EAGER)


def current_mode() -> Mode:
    return _MODE.get()


@contextlib.contextmanager
def graph_capture():
    """``with graph_capture(), torch.cuda.graph(g): ...`` marks the scope as capture."""
    token = _MODE.set(Mode.GRAPH_CAPTURING)
    try:
        yield
    finally:
        _MODE.reset(token)


class NoBackendError(Exception):
    """No registered linear kernel can take the requested (spec, shape, mode).

    Same role as ``phyai/parallel/exceptions.py:14-15`` in the reference.
    """


__all__ = ["Mode", "current_mode", "graph_capture", "NoBackendError"]
