"""Helpers for tests in the reference's style: run a function through the
backend, compare with eager, and assert on the pass log
(reference src/xpu_graph/test_utils.py:13-14,105-130)."""
import contextlib
import logging

import torch


def is_similar(result, expected, rtol=0.01, atol=0.01):
    return result.shape == expected.shape and torch.allclose(result, expected, rtol, atol)


def maybe_similar(result, expected, rtol=0.01, atol=0.01):
    if result is None or expected is None:
        return result is None and expected is None
    return is_similar(result, expected, rtol, atol)


@contextlib.contextmanager
def need_xpu_graph_logs():
    """Let pytest's caplog see the DEBUG log of the pass pipeline."""
    lg = logging.getLogger("xpu_graph")
    saved = (lg.propagate, lg.level)
    lg.propagate = True
    lg.setLevel(logging.DEBUG)
    try:
        yield
    finally:
        lg.propagate, _ = saved
        lg.setLevel(saved[1])


@contextlib.contextmanager
def skip_xpu_graph_cache(backend):
    """Force recompilation: Dynamo's code cache is reset and the backend's artifact cache is swapped for the base
    class, which stores nothing (reference test_utils.py:120-130)."""
    from .cache import XpuGraphCache

    saved = backend._cache
    try:
        torch._dynamo.reset_code_caches()
        backend._cache = XpuGraphCache() if saved is not None else None
        yield
    finally:
        backend._cache = saved
