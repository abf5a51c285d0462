"""One helper thread on which all device work of the planner runs.

The planner is usually called while a graph-capture context keeps a FakeTensorMode (or
another dispatch mode) active in the caller's thread (the reference builds its optimizer
inside ``AutoParallel.__enter__``, api.py:273-282): a tensor made there would be a fake one
and an operator would be handed fakes.  torch keeps its dispatch modes per thread, so code
that runs on a thread of its own sees none of them and its tensors are real allocations,
without reaching into torch's private mode stack.  The caller's current stream (also
per-thread state) is carried over, so "the current stream" keeps meaning the caller's.

Calls are serialised (one worker), nested calls run in place, exceptions come back to the
caller unchanged.
"""

from __future__ import annotations

import functools
import os
import threading
from concurrent.futures import ThreadPoolExecutor

_lock = threading.Lock()
_pool: ThreadPoolExecutor | None = None
_worker_ident: int | None = None


def _remember_ident():
    global _worker_ident
    _worker_ident = threading.get_ident()


def _executor() -> ThreadPoolExecutor:
    global _pool
    with _lock:
        if _pool is None:
            _pool = ThreadPoolExecutor(max_workers=1, thread_name_prefix="apcost-device",
                                       initializer=_remember_ident)
        return _pool


def _forget_thread():
    # a forked child has the parent's pool object but none of its threads
    global _pool, _worker_ident
    _pool = None
    _worker_ident = None


os.register_at_fork(after_in_child=_forget_thread)


def _callers_stream():
    """The caller's current stream, None on a machine without a GPU.  A child forked from a
    process that had already initialised the GPU cannot use the device at all (torch refuses
    to initialise it a second time): that is reported as what it is, not as a torch internal."""
    import torch

    if not torch.cuda.is_available():
        return None
    try:
        return torch.cuda.current_stream()
    except RuntimeError as e:
        if "fork" in str(e):
            raise RuntimeError("apcost: this process was forked from one that had initialised the GPU; a forked child "
                               "cannot do device work (start workers with the 'spawn' method, or fork before the "
                               "parent touches the GPU)") from e
        raise


def call(fn, *args, **kwargs):
    """``fn(*args, **kwargs)`` on the device thread; the result (or the exception) of the call.
    In a forked child the parent's thread is gone and the first call starts a new one; device
    work there needs a parent that had not initialised the GPU before the fork."""
    if threading.get_ident() == _worker_ident:
        return fn(*args, **kwargs)
    import torch

    stream = _callers_stream()

    def task():
        if stream is None:
            return fn(*args, **kwargs)
        with torch.cuda.stream(stream):  # (sets the stream's device as well)
            return fn(*args, **kwargs)

    return _executor().submit(task).result()


def submit(fn, *args, **kwargs):
    """Queues ``fn(*args, **kwargs)`` on the device thread and returns its future without
    waiting (work that may overlap the caller's: the device's first-use costs)."""
    return _executor().submit(fn, *args, **kwargs)


def on_device_thread(fn):
    """Decorator form of ``call``."""

    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        return call(fn, *args, **kwargs)

    return wrapper
